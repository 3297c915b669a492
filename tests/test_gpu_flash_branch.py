"""The layer's flash branch (the reference's ``_flash_attention`` and the
dispatch in ``forward``, ironcore/layers/attention.py:144-206,230-250) on the
GPU kernels.

The flash-attn wheel is absent here, so nothing below compares with it.  What
pins the branch is what the reference's own tests say it must equal
(tests/test_attention.py:618-789: the flash layer called with no mask against
the dense layer called with the causal mask, MHA and GQA, loose bars mean < 0.1
and max < 1.0) and flash-attn's published alignment of the causal rule for
sq != sk (bottom right).  Held here to the oracle's dense attention under that
mask, at the kernels' own bar."""
import pytest
import torch

from ironcore_amd import config as ic_config
from ironcore_amd.layers import Attention
from ironcore_amd.layers import attention as attention_module
from oracle.dense_attention import causal_offset_mask, dense_attention

pytestmark = pytest.mark.gpu


def _cfg(heads, groups, hd, precision, flash, dropout=0.0):
    return ic_config.MainConfig(model=ic_config.ModelConfig(
        d_model=heads * hd, num_attention_heads=heads, num_attention_groups=groups, head_dim=hd,
        dropout_attn=dropout, precision=precision), trainer=ic_config.TrainerConfig(use_flash_attn=flash))


def _qkv(b, sq, sk, hn, gn, hd, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(b, sq, hn, hd, generator=g).to(dtype), torch.randn(b, sk, gn, hd, generator=g).to(dtype),
            torch.randn(b, sk, gn, hd, generator=g).to(dtype))


@pytest.fixture
def wheel_present(monkeypatch):
    """The reference takes the branch when the wheel's import worked; the name
    is only that switch here (the wheel itself is never called)."""
    def never_called(*a, **k):
        raise AssertionError("the flash branch must run on this package's kernels")
    monkeypatch.setattr(attention_module, "flash_attn_varlen_func", never_called)


@pytest.mark.parametrize("dtype,precision,tol", [(torch.bfloat16, "bf16", 2e-2), (torch.float16, "fp16", 2e-2),
                                                 (torch.float32, "fp32", 1e-4)])
@pytest.mark.parametrize("hn,gn", [(8, 8), (8, 2), (8, 1)])
def test_flash_layer_without_mask_equals_dense_layer_with_causal_mask(gpu, wheel_present, dtype, precision, tol, hn, gn):
    """The reference's three comparisons (MHA :618-671, GQA :673-730, MQA
    :732-789): batch 2, 64 tokens, 8 heads of 64."""
    b, s, hd = 2, 64, 64
    q, k, v = _qkv(b, s, s, hn, gn, hd, dtype, seed=42 + gn)
    mask = torch.tril(torch.ones(s, s)).view(1, 1, s, s).expand(b, -1, -1, -1)
    want = dense_attention(q, k, v, mask)
    flash = Attention(_cfg(hn, gn, hd, precision, flash=True)).to(gpu).eval()
    dense = Attention(_cfg(hn, gn, hd, precision, flash=False)).to(gpu).eval()
    got_flash = flash(q.to(gpu), k.to(gpu), v.to(gpu), None).cpu().float()
    got_dense = dense(q.to(gpu), k.to(gpu), v.to(gpu), mask.to(gpu)).cpu().float()
    diff = (got_flash - got_dense).abs()
    assert diff.mean().item() < 0.1 and diff.max().item() < 1.0   # the reference's bars
    assert torch.equal(got_flash, got_dense)                       # here: the same kernel, the same launch
    assert (got_flash - want.float()).abs().max().item() <= tol


def test_flash_branch_ignores_the_mask_and_needs_the_switch(gpu, monkeypatch):
    """forward: the branch is taken when the config asks for it AND the wheel's
    import worked; it then ignores attention_mask (attention.py:230,240-250).
    Without the wheel the same config runs the dense branch with the mask."""
    b, s, hn, hd = 2, 48, 4, 64
    q, k, v = _qkv(b, s, s, hn, hn, hd, torch.bfloat16, seed=3)
    window = (torch.arange(s).view(-1, 1) - torch.arange(s).view(1, -1)).abs() <= 2   # neither causal nor full
    mask = window.float().view(1, 1, s, s)
    layer = Attention(_cfg(hn, hn, hd, "bf16", flash=True)).to(gpu).eval()
    causal = dense_attention(q, k, v, causal_offset_mask(s, s))
    banded = dense_attention(q, k, v, mask)
    monkeypatch.setattr(attention_module, "flash_attn_varlen_func", None)
    got = layer(q.to(gpu), k.to(gpu), v.to(gpu), mask.to(gpu)).cpu().float()
    assert (got - banded.float()).abs().max().item() <= 2e-2
    monkeypatch.setattr(attention_module, "flash_attn_varlen_func", lambda *a, **k: None)
    got = layer(q.to(gpu), k.to(gpu), v.to(gpu), mask.to(gpu)).cpu().float()
    assert (got - causal.float()).abs().max().item() <= 2e-2
    assert (got - banded.float()).abs().max().item() > 0.1


@pytest.mark.parametrize("sq,sk", [(17, 90), (64, 64), (1, 33), (90, 17)])
@pytest.mark.parametrize("causal", [True, False])
def test_flash_attention_method_alignment(gpu, sq, sk, causal):
    """_flash_attention called as the reference calls it (:240-250), for sq != sk
    too: the causal rule sits at the bottom right (row i sees keys
    j <= (sk - sq) + i); rows above the triangle (sq > sk) see nothing and
    return zeros."""
    b, hn, gn, hd = 2, 6, 3, 128
    q, k, v = _qkv(b, sq, sk, hn, gn, hd, torch.bfloat16, seed=sq * 100 + sk)
    layer = Attention(_cfg(hn, gn, hd, "bf16", flash=True)).to(gpu).eval()
    got = layer._flash_attention(q.to(gpu), k.to(gpu), v.to(gpu), sq, sk, sq, sk, causal=causal).cpu().float()
    assert got.shape == (b, sq, hn * hd)
    if not causal:
        want = dense_attention(q, k, v, None).float()
        assert (got - want).abs().max().item() <= 2e-2
        return
    top = max(sq - sk, 0)
    assert torch.count_nonzero(got[:, :top]) == 0
    want = dense_attention(q[:, top:], k, v, causal_offset_mask(sq - top, sk)).float()
    assert (got[:, top:] - want).abs().max().item() <= 2e-2


def test_flash_attention_method_refuses_what_is_not_built(gpu):
    q, k, v = (t.to(gpu) for t in _qkv(1, 8, 8, 2, 2, 64, torch.bfloat16, seed=0))
    layer = Attention(_cfg(2, 2, 64, "bf16", flash=True)).to(gpu).eval()
    with pytest.raises(NotImplementedError, match="sliding-window"):
        layer._flash_attention(q, k, v, 8, 8, 8, 8, causal=True, window_size=(4, 0))
    with pytest.raises(NotImplementedError, match="ALiBi"):
        layer._flash_attention(q, k, v, 8, 8, 8, 8, alibi_slopes=torch.ones(2, device=gpu))
    with pytest.raises(ValueError, match="do not match"):
        layer._flash_attention(q, k, v, 8, 9, 8, 9)
    wet = Attention(_cfg(2, 2, 64, "bf16", flash=True, dropout=0.1)).to(gpu).eval()
    with pytest.raises(NotImplementedError, match="dropout"):
        wet._flash_attention(q, k, v, 8, 8, 8, 8, causal=True)
