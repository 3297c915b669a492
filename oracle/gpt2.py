"""CPU restatement of the reference's decoder forward (GPT-2 and Llama
shaped) and of the two generate loops (TEST INFRASTRUCTURE, not product code).

Weights come in as a plain ``{name: tensor}`` dict using the reference's
parameter names (``embedding.word_embeddings.weight``, ``model.layers.N.
linear_q.weight`` ..., weights stored ``[in, out]``).  The arithmetic follows

    ironcore/language_model.py:67-100,102-161,203-227   masks, positions, logits
    ironcore/layers/embedding.py:34-50                  word + learned position
    ironcore/models/transformer.py:77-132               pre-LN block
    ironcore/layers/mlp.py:48-54                        up -> activation -> down
    ironcore/layers/activations/activations.py:26-39    glu / swiglu gating
    ironcore/layers/layernorm/fused_layer_norm.py:24-28 nn.LayerNorm
    ironcore/layers/layernorm/fused_rms_norm.py:19-28   nn.RMSNorm (scale only)
    ironcore/parallel/tensor_parallel/layers.py:194-204,250-263   x @ W + b
    ironcore/layers/attention.py:68-142                 (via dense_attention)

``generate_full_recompute`` is the reference's loop
(examples/generate_text.py:24-40) with greedy selection; ``generate_paged``
is the same model driven through a block KV cache.  For a causal model the two
must pick from identical last-position logits (up to float reassociation),
which is what pins the cached loop without any reference import.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from . import paged as oracle_paged
from .dense_attention import causal_offset_mask, dense_attention
from .rope import rope_rotate


class Dims:
    def __init__(self, num_layers, num_heads, num_groups, d_model, ln_eps=1e-5, post_ln=False, rope=None,
                 ln_type="layernorm", activation="gelu"):
        """``rope``: (cos_table, sin_table) when query and key rows are rotated
        (transformer.py:95-98) at their index in the sequence, else None.
        ``ln_type``: layernorm | rmsnorm.  ``activation``: gelu | relu | silu |
        glu | swiglu."""
        self.rope = rope
        self.ln_type = ln_type
        self.activation = activation
        self.num_layers = num_layers
        self.num_heads = num_heads
        self.num_groups = num_groups
        self.d_model = d_model
        self.head_dim = d_model // num_heads
        self.ln_eps = ln_eps
        self.post_ln = post_ln


def _linear(x, w, name):
    y = torch.matmul(x, w[name + ".weight"])
    bias = w.get(name + ".bias")
    return y + bias if bias is not None else y


def _norm(x, w, name, eps, ln_type="layernorm"):
    if ln_type == "rmsnorm":  # x / sqrt(mean(x^2) + eps) * scale, written out
        xf = x.float()
        y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
        return (y * w[name + ".layernorm.weight"].float()).to(x.dtype)
    return F.layer_norm(x, (x.shape[-1],), w[name + ".layernorm.weight"], w.get(name + ".layernorm.bias"), eps)


def _activate(x, kind):
    if kind == "gelu":
        return F.gelu(x)
    if kind == "relu":
        return F.relu(x)
    if kind == "silu":
        return F.silu(x)
    feature, gate = x.chunk(2, dim=-1)  # activations.py:28
    if kind == "glu":
        return feature * torch.sigmoid(gate)
    if kind == "swiglu":
        return F.silu(feature) * gate
    raise NotImplementedError(kind)


def _embed(w, input_ids, pos):
    x = F.embedding(input_ids, w["embedding.word_embeddings.weight"])
    if "embedding.position_embedding.weight" in w:  # embedding.py:16: learned positions only when "absolute"
        x = x + F.embedding(pos, w["embedding.position_embedding.weight"])
    return x


def _rotate(x, pos, dims):
    """rotary.py:69-83 on rows [b, s, heads, hd] at positions [b, s]; the rows
    keep the model dtype (what a cache of that dtype stores)."""
    b, s, h, d = x.shape
    out = rope_rotate(x.reshape(b * s, h, d), pos.reshape(-1), dims.rope[0], dims.rope[1])
    return out.to(x.dtype).view(b, s, h, d)


def _layer(x, w, prefix, dims, attend, pos=None):
    """One transformer block; `attend(q, k, v)` supplies the attention result
    for q [b,s,hn,hd], k/v [b,s,gn,hd] (the new tokens' rows); with rotary
    embeddings q and k are rotated at `pos` [b, s] first."""
    b, s, _ = x.shape
    norm_out = _norm(x, w, prefix + "input_layernorm", dims.ln_eps, dims.ln_type)
    q = _linear(norm_out, w, prefix + "linear_q")
    k, v = torch.chunk(_linear(norm_out, w, prefix + "linear_kv"), 2, dim=-1)
    q = q.view(b, s, dims.num_heads, dims.head_dim)
    k = k.view(b, s, dims.num_groups, dims.head_dim)
    v = v.view(b, s, dims.num_groups, dims.head_dim)
    if dims.rope is not None:
        q, k = _rotate(q, pos, dims), _rotate(k, pos, dims)
    attn = _linear(attend(q, k, v), w, prefix + "attn_output")
    residual = norm_out if dims.post_ln else x
    norm_in = residual + attn
    norm_out = _norm(norm_in, w, prefix + "post_attn_layernorm", dims.ln_eps, dims.ln_type)
    mlp = _linear(_activate(_linear(norm_out, w, prefix + "mlp.up_proj"), dims.activation), w,
                  prefix + "mlp.down_proj")
    residual = norm_out if dims.post_ln else norm_in
    return residual + mlp


def _logits(x, w, dims):
    x = _norm(x, w, "output_layernorm", dims.ln_eps, dims.ln_type)
    if "output_layer.weight" in w:
        return torch.matmul(x, w["output_layer.weight"])
    return torch.matmul(x, w["embedding.word_embeddings.weight"].transpose(0, 1))


def forward_full(w, dims, input_ids):
    """Full causal pass: logits [b, s, vocab] (language_model.py:67-100 with labels=None)."""
    b, s = input_ids.shape
    mask = torch.tril(torch.ones(s, s)).view(1, 1, s, s) > 0.5
    pos = torch.arange(s).unsqueeze(0).expand(b, s)
    x = _embed(w, input_ids, pos)
    for i in range(dims.num_layers):
        x = _layer(x, w, f"model.layers.{i}.", dims, lambda q, k, v: dense_attention(q, k, v, mask), pos)
    return _logits(x, w, dims)


@torch.no_grad()
def generate_full_recompute(w, dims, input_ids, max_new_tokens, return_margins=False):
    tokens = input_ids
    margins = []
    for _ in range(max_new_tokens):
        logits = forward_full(w, dims, tokens)[:, -1, :]
        if return_margins:
            top2 = torch.topk(logits.float(), 2, dim=-1)[0]
            margins.append(top2[:, 0] - top2[:, 1])
        tokens = torch.cat([tokens, logits.argmax(dim=-1, keepdim=True)], dim=1)
    return (tokens, torch.stack(margins, 1)) if return_margins else tokens


class OracleCache:
    """Minimal block KV cache for the oracle loop: identity-free allocation in
    a shuffled block order, one table per sequence, pools per layer."""

    def __init__(self, dims, batch, max_len, block_size, dtype, seed=0):
        per_seq = (max_len + block_size - 1) // block_size
        n = batch * per_seq
        order = torch.randperm(n, generator=torch.Generator().manual_seed(seed))
        self.block_size = block_size
        self.tables = order.view(batch, per_seq).to(torch.int32)
        self.lens = [0] * batch
        shape = (n, dims.num_groups, block_size, dims.head_dim)
        self.k = [torch.zeros(shape, dtype=dtype) for _ in range(dims.num_layers)]
        self.v = [torch.zeros(shape, dtype=dtype) for _ in range(dims.num_layers)]

    def slots_for(self, n_new):
        bs = self.block_size
        slots = []
        for i, have in enumerate(self.lens):
            for t in range(have, have + n_new):
                slots.append(int(self.tables[i, t // bs]) * bs + t % bs)
        return torch.tensor(slots, dtype=torch.int64)


def forward_paged(w, dims, cache, new_ids):
    """New tokens [b, s] of sequences living in `cache`: append their K/V,
    attend against the cache, return logits [b, s, vocab]."""
    b, s = new_ids.shape
    past = torch.tensor(cache.lens)
    pos = past.unsqueeze(1) + torch.arange(s).unsqueeze(0)
    slots = cache.slots_for(s)
    ctx = torch.tensor([l + s for l in cache.lens], dtype=torch.int32)
    cu = torch.arange(0, (b + 1) * s, s, dtype=torch.int32)
    x = _embed(w, new_ids, pos)
    for i in range(dims.num_layers):
        def attend(q, k, v, i=i):
            oracle_paged.kv_append(cache.k[i], cache.v[i], k.reshape(b * s, dims.num_groups, dims.head_dim),
                                   v.reshape(b * s, dims.num_groups, dims.head_dim), slots)
            out = oracle_paged.paged_prefill(q.reshape(b * s, dims.num_heads, dims.head_dim), cache.k[i],
                                             cache.v[i], cache.tables, ctx, cu)
            return out.view(b, s, -1)
        x = _layer(x, w, f"model.layers.{i}.", dims, attend, pos)
    cache.lens = [l + s for l in cache.lens]
    return _logits(x, w, dims)


@torch.no_grad()
def generate_paged(w, dims, input_ids, max_new_tokens, block_size=16, return_margins=False):
    b, s = input_ids.shape
    dtype = w["embedding.word_embeddings.weight"].dtype
    cache = OracleCache(dims, b, s + max_new_tokens, block_size, dtype)
    tokens = input_ids
    step = input_ids
    margins = []
    for _ in range(max_new_tokens):
        logits = forward_paged(w, dims, cache, step)[:, -1, :]
        if return_margins:
            top2 = torch.topk(logits.float(), 2, dim=-1)[0]
            margins.append(top2[:, 0] - top2[:, 1])
        step = logits.argmax(dim=-1, keepdim=True)
        tokens = torch.cat([tokens, step], dim=1)
    return (tokens, torch.stack(margins, 1)) if return_margins else tokens
