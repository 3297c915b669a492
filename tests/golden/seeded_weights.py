"""Deterministic weights for the golden fixtures: every tensor of a Hugging
Face GPT-2 / Llama state dict drawn from numpy's PCG64 stream in a fixed
(sorted-name) order, so that the fixture files need to hold only the seed,
the inputs and the expected outputs.  Used by make_fixtures.py (which feeds
the tensors to transformers) and by tests/test_golden.py (which feeds the same
tensors to this repository's loaders)."""
from __future__ import annotations

import numpy as np
import torch

GPT2 = dict(vocab=300, n_pos=64, d=128, heads=2, layers=2, eps=1e-5)
LLAMA = dict(vocab=300, n_pos=64, d=256, heads=4, groups=2, ffn=320, layers=2, eps=1e-5, theta=10000.0)


def _draw(shapes, seed):
    rng = np.random.default_rng(seed)
    out = {}
    for name in sorted(shapes):
        x = rng.standard_normal(shapes[name]).astype(np.float32) * 0.05
        if "ln_" in name or "norm" in name:
            x = x + (1.0 if name.endswith("weight") else 0.0)   # norm scales around 1, norm biases around 0
        out[name] = torch.from_numpy(x)
    return out


def gpt2_state(seed: int):
    c = GPT2
    d = c["d"]
    shapes = {"wte.weight": (c["vocab"], d), "wpe.weight": (c["n_pos"], d), "ln_f.weight": (d,), "ln_f.bias": (d,)}
    for i in range(c["layers"]):
        p = f"h.{i}."
        shapes.update({p + "ln_1.weight": (d,), p + "ln_1.bias": (d,), p + "ln_2.weight": (d,), p + "ln_2.bias": (d,),
                       p + "attn.c_attn.weight": (d, 3 * d), p + "attn.c_attn.bias": (3 * d,),
                       p + "attn.c_proj.weight": (d, d), p + "attn.c_proj.bias": (d,),
                       p + "mlp.c_fc.weight": (d, 4 * d), p + "mlp.c_fc.bias": (4 * d,),
                       p + "mlp.c_proj.weight": (4 * d, d), p + "mlp.c_proj.bias": (d,)})
    return _draw(shapes, seed)


def llama_state(seed: int):
    c = LLAMA
    d, hd = c["d"], c["d"] // c["heads"]
    shapes = {"model.embed_tokens.weight": (c["vocab"], d), "model.norm.weight": (d,), "lm_head.weight": (c["vocab"], d)}
    for i in range(c["layers"]):
        p = f"model.layers.{i}."
        shapes.update({p + "input_layernorm.weight": (d,), p + "post_attention_layernorm.weight": (d,),
                       p + "self_attn.q_proj.weight": (c["heads"] * hd, d),
                       p + "self_attn.k_proj.weight": (c["groups"] * hd, d),
                       p + "self_attn.v_proj.weight": (c["groups"] * hd, d),
                       p + "self_attn.o_proj.weight": (d, c["heads"] * hd),
                       p + "mlp.gate_proj.weight": (c["ffn"], d), p + "mlp.up_proj.weight": (c["ffn"], d),
                       p + "mlp.down_proj.weight": (d, c["ffn"])})
    return _draw(shapes, seed)
