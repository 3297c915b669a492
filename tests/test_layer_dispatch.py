"""Which branch Attention.forward takes (host logic, no GPU): the reference's
rule (ironcore/layers/attention.py:230): the flash branch when the config asks
for it and the flash-attn import worked, else the dense branch with the mask."""
import torch

from ironcore_amd import config as ic_config
from ironcore_amd.layers import Attention
from ironcore_amd.layers import attention as attention_module


def _layer(flash):
    cfg = ic_config.MainConfig(model=ic_config.ModelConfig(
        d_model=128, num_attention_heads=2, num_attention_groups=2, head_dim=64, dropout_attn=0.0,
        precision="bf16"), trainer=ic_config.TrainerConfig(use_flash_attn=flash))
    return Attention(cfg).eval()


def _calls(layer, monkeypatch):
    seen = []
    monkeypatch.setattr(layer, "_dense", lambda q, k, v, m: seen.append(("dense", m)) or "dense")
    monkeypatch.setattr(layer, "_flash_attention",
                        lambda q, k, v, sq, sk, mq, mk, causal=False, window_size=(-1, -1), alibi_slopes=None:
                        seen.append(("flash", sq, sk, mq, mk, causal, tuple(window_size), alibi_slopes)) or "flash")
    return seen


def test_branch_follows_config_and_import(monkeypatch):
    q = torch.zeros(1, 5, 2, 64, dtype=torch.bfloat16)
    kv = torch.zeros(1, 9, 2, 64, dtype=torch.bfloat16)
    mask = torch.ones(1, 1, 5, 9)
    for flash_cfg, wheel, want in [(True, object(), "flash"), (True, None, "dense"), (False, object(), "dense"),
                                   (False, None, "dense")]:
        monkeypatch.setattr(attention_module, "flash_attn_varlen_func", wheel)
        layer = _layer(flash_cfg)
        seen = _calls(layer, monkeypatch)
        assert layer(q, kv, kv, mask) == want
        if want == "flash":   # causal, whole sequences, no window, the mask not handed over (attention.py:240-250)
            assert seen == [("flash", 5, 9, 5, 9, True, (-1, -1), None)]
        else:
            assert seen == [("dense", mask)]
