"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py).

Expected values come from implementations that share no code with the oracle
or the kernels: float64 loops for attention, the transformers package for the
GPT-2 and Llama forwards.  The CPU tests hold the oracle to them; the GPU
tests hold the HIP path (through the attention layer, the model and the cached
generate loop) to them.  Neither needs transformers at run time: weights are
re-drawn from the fixture's seed."""
import json
import pathlib
import sys

import numpy as np
import pytest
import torch

from ironcore_amd import config as ic_config
from ironcore_amd import generation, weights

GOLDEN = pathlib.Path(__file__).resolve().parent / "golden"
sys.path.insert(0, str(GOLDEN))
import seeded_weights as sw  # noqa: E402

ATTENTION_CASES = ["mha_causal", "gqa_chunk", "decode"]


def _attention_case(name):
    d = np.load(GOLDEN / "attention_f64.npz")
    mask = torch.from_numpy(d[name + "_mask"]).unsqueeze(1) if name + "_mask" in d else None   # [b or 1, 1, sq, sk]
    return (torch.from_numpy(d[name + "_q"]), torch.from_numpy(d[name + "_k"]), torch.from_numpy(d[name + "_v"]),
            mask, torch.from_numpy(d[name + "_out"]))


@pytest.mark.parametrize("name", ATTENTION_CASES)
def test_oracle_attention_against_float64_loops(name):
    from oracle.dense_attention import dense_attention
    q, k, v, mask, want = _attention_case(name)
    got = dense_attention(q, k, v, mask)
    assert (got.double() - want).abs().max().item() < 2e-6
    got16 = dense_attention(q.bfloat16(), k.bfloat16(), v.bfloat16(), mask)
    assert (got16.double() - want).abs().max().item() < 2e-2                   # the bf16 bar, on the same numbers


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-2), (torch.float16, 4e-3)])
@pytest.mark.parametrize("name", ATTENTION_CASES)
def test_attention_layer_against_float64_loops(gpu, name, dtype, tol):
    from ironcore_amd.layers import Attention
    q, k, v, mask, want = _attention_case(name)
    hn, gn, hd = q.shape[2], k.shape[2], q.shape[3]
    precision = {torch.float32: "fp32", torch.bfloat16: "bf16", torch.float16: "fp16"}[dtype]
    cfg = ic_config.MainConfig(model=ic_config.ModelConfig(d_model=hn * hd, num_attention_heads=hn,
                                                           num_attention_groups=gn, head_dim=hd, dropout_attn=0.0,
                                                           precision=precision),
                               trainer=ic_config.TrainerConfig(use_flash_attn=False))
    layer = Attention(cfg).to(gpu).eval()
    if name == "gqa_chunk":
        # the layer takes the causal mask of a chunk that ends the sequence, or none: this is that mask
        assert bool((mask[0, 0, -1] != 0).all())
    out = layer(q.to(gpu, dtype), k.to(gpu, dtype), v.to(gpu, dtype), None if mask is None else mask.to(gpu))
    torch.cuda.synchronize()
    assert (out.cpu().double() - want).abs().max().item() < tol


def _gpt2(precision="fp32"):
    d = np.load(GOLDEN / "gpt2_transformers.npz")
    c = json.loads(str(d["config"]))
    cfg = ic_config.MainConfig(
        model=ic_config.ModelConfig(d_model=c["d"], d_ffn=4 * c["d"], num_layers=c["layers"],
                                    num_attention_heads=c["heads"], head_dim=c["d"] // c["heads"],
                                    max_seq_len=c["n_pos"], max_position_embeddings=c["n_pos"], dropout_attn=0.0,
                                    dropout_embd=0.0, dropout_mlp=0.0, precision=precision, ln_eps=c["eps"],
                                    activation_type="gelu"),
        trainer=ic_config.TrainerConfig(use_flash_attn=False))
    model = generation.LanguageModel(cfg, vocab_size=c["vocab"])
    weights.load_hf_gpt2(model, sw.gpt2_state(int(d["seed"])))
    return model, cfg, c, d


def _llama(precision="fp32"):
    d = np.load(GOLDEN / "llama_transformers.npz")
    c = json.loads(str(d["config"]))
    cfg = ic_config.MainConfig(
        model=ic_config.ModelConfig(d_model=c["d"], d_ffn=c["ffn"], num_layers=c["layers"],
                                    num_attention_heads=c["heads"], num_attention_groups=c["groups"],
                                    head_dim=c["d"] // c["heads"], max_seq_len=c["n_pos"],
                                    max_position_embeddings=c["n_pos"], dropout_attn=0.0, dropout_embd=0.0,
                                    dropout_mlp=0.0, precision=precision, ln_eps=c["eps"], ln_type="rmsnorm",
                                    activation_type="swiglu", no_bias=True, untie_embed=True,
                                    positional_embedding=ic_config.PositionalEmbeddingConfig(type="rope",
                                                                                             base=int(c["theta"]))),
        trainer=ic_config.TrainerConfig(use_flash_attn=False))
    model = generation.LanguageModel(cfg, vocab_size=c["vocab"])
    weights.load_hf_llama(model, sw.llama_state(int(d["seed"])))
    return model, cfg, c, d


def _oracle_dims(cfg, kind):
    from oracle import gpt2 as oracle_gpt2
    from oracle.rope import rope_tables
    m = cfg.model
    if kind == "gpt2":
        return oracle_gpt2.Dims(m.num_layers, m.num_attention_heads, m.num_attention_groups, m.d_model, m.ln_eps)
    rope = rope_tables(m.d_model // m.num_attention_heads, m.max_position_embeddings, m.positional_embedding.base)
    return oracle_gpt2.Dims(m.num_layers, m.num_attention_heads, m.num_attention_groups, m.d_model, m.ln_eps,
                            rope=rope, ln_type="rmsnorm", activation="swiglu")


@pytest.mark.parametrize("kind", ["gpt2", "llama"])
def test_oracle_model_against_transformers_fixture(kind):
    from oracle import gpt2 as oracle_gpt2
    model, cfg, c, d = _gpt2() if kind == "gpt2" else _llama()
    w = {k: v.detach().clone() for k, v in model.state_dict().items() if not k.startswith("rotary_pos_emb.")}
    dims = _oracle_dims(cfg, kind)
    ids = torch.from_numpy(d["ids"])
    got = oracle_gpt2.forward_full(w, dims, ids)[..., :c["vocab"]]
    assert (got - torch.from_numpy(d["logits"])).abs().max().item() < 1e-4
    tokens = torch.from_numpy(d["tokens"])
    assert float(d["min_margin"]) > 5e-3                                        # no step of the fixture is a near tie
    assert torch.equal(oracle_gpt2.generate_paged(w, dims, tokens[:, :9], tokens.shape[1] - 9), tokens)
    assert torch.equal(oracle_gpt2.generate_full_recompute(w, dims, tokens[:, :9], tokens.shape[1] - 9), tokens)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["gpt2", "llama"])
def test_gpu_model_against_transformers_fixture(gpu, kind):
    model, cfg, c, d = _gpt2() if kind == "gpt2" else _llama()
    model = model.to(gpu).eval()
    ids = torch.from_numpy(d["ids"]).to(gpu)
    with torch.no_grad():
        got = model(ids)[..., :c["vocab"]].cpu()
    assert (got - torch.from_numpy(d["logits"])).abs().max().item() < 1e-4
    tokens = torch.from_numpy(d["tokens"])
    ours = generation.generate(model, tokens[:, :9].to(gpu), tokens.shape[1] - 9)
    torch.cuda.synchronize()
    assert torch.equal(ours.cpu(), tokens)
