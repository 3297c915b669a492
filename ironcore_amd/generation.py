"""Generation through the block KV cache: the model-side callers of the
attention layer and the generate loop.

The reference reaches its attention layer only through
``LanguageModel.forward`` -> ``TransformerModel`` -> ``TransformerLayer.
custom_forward`` (ironcore/language_model.py:67-100, ironcore/models/
transformer.py:77-162) and generates by re-running that forward on the whole
growing sequence every step (examples/generate_text.py:12-46).  The classes
below keep that arithmetic and those parameter names, add the two optional
arguments that carry the KV cache down to ``Attention.forward``, and replace
the full recompute by prefill + cached decode.  The GEMMs, norms and the
activation are plain torch calls on the GPU (plumbing around the hot path);
attention and the KV append are the HIP kernels.

Built: pre/post-LN with LayerNorm or RMSNorm, learned absolute positions or
rotary embeddings, GELU/ReLU/SiLU and gated (GLU/SwiGLU/GeGLU/SiGLU) MLPs, tied or
untied output embedding: the GPT-2 and the Llama family of shapes.  Rotary embeddings use each
token's index in its sequence; the reference's rotary module picks the angle
of a row by its batch index (ironcore/layers/positional_embedding/
rotary.py:53-64), which no KV-cached path can reproduce meaningfully (see
layers/rotary.py).
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch
import torch.nn.functional as F
from torch import nn

from .kv_cache import PagedKVCache
from .layers.attention import Attention, PagedAttentionMetadata
from .layers.module import BaseModule, get_model_dtype
from .layers.rotary import RotaryPositionalEmbedding


class Linear(BaseModule):
    """``y = x @ W + b`` with the weight stored ``[in, out]`` as the reference's
    parallel linears do at tensor-parallel size 1
    (ironcore/parallel/tensor_parallel/layers.py:41,194-204,250-263)."""

    def __init__(self, config, input_size: int, output_size: int, bias: bool):
        super().__init__(config)
        self.weight = nn.Parameter(torch.empty(input_size, output_size))
        self.bias = nn.Parameter(torch.empty(output_size)) if bias else None

    def forward(self, x):
        y = torch.matmul(x, self.weight)
        return y + self.bias if self.bias is not None else y


class LayerNorm(BaseModule):
    """ironcore/layers/layernorm/fused_layer_norm.py:20-28 (wraps nn.LayerNorm)."""

    def __init__(self, config):
        super().__init__(config)
        self.layernorm = nn.LayerNorm(config.model.d_model, eps=config.model.ln_eps,
                                      bias=not config.model.no_bias)

    def forward(self, x):
        return self.layernorm(x)


class RmsNorm(BaseModule):
    """ironcore/layers/layernorm/fused_rms_norm.py:19-28: ``nn.RMSNorm`` under
    the attribute ``layernorm``.  The reference also passes ``bias=`` to it,
    which torch's RMSNorm does not take (it has a scale only), so that
    constructor call fails there; here the scale alone is created."""

    def __init__(self, config):
        super().__init__(config)
        self.layernorm = nn.RMSNorm(config.model.d_model, eps=config.model.ln_eps)

    def forward(self, x):
        return self.layernorm(x)


def get_layernorm(config) -> nn.Module:
    """ironcore/layers/layernorm/__init__.py:18-26."""
    kind = config.model.ln_type.lower()
    if kind == "layernorm":
        return LayerNorm(config)
    if kind == "rmsnorm":
        return RmsNorm(config)
    raise NotImplementedError(f"{kind} is not supported")


class GLUActivation(nn.Module):
    """ironcore/layers/activations/activations.py:15-42.  The input is the
    ``[feature | gate]`` concatenation the doubled up-projection produces;
    ``swiglu`` is ``silu(feature) * gate``, so in Llama terms the first half of
    the up-projection is ``gate_proj`` and the second ``up_proj``."""

    def __init__(self, input_dim: int, variant: str = "glu"):
        super().__init__()
        self.variant = variant.lower()
        if self.variant not in ("glu", "geglu", "siglu", "swiglu"):
            raise ValueError(f"Unknown GLU variant: {self.variant}")
        if self.variant in ("geglu", "siglu"):
            self.linear = nn.Linear(input_dim, input_dim)

    def forward(self, x):
        feature, gate = x.chunk(2, dim=-1)
        if self.variant == "glu":
            return feature * torch.sigmoid(gate)
        if self.variant == "geglu":
            return self.linear(feature) * torch.sigmoid(gate)
        if self.variant == "siglu":
            return feature * torch.sigmoid(self.linear(gate))
        return F.silu(feature) * gate


def get_activation(name: str, input_dim: Optional[int] = None) -> nn.Module:
    """ironcore/layers/activations/activations.py:45-60."""
    if name == "relu":
        return nn.ReLU()
    if name == "gelu":
        return nn.GELU()
    if name == "silu":
        return nn.SiLU()
    if "glu" in name:
        if input_dim is None:
            raise ValueError("input_dim is required for GLU activation")
        return GLUActivation(input_dim, name)
    raise NotImplementedError(f"activation {name!r}")


class MLP(BaseModule):
    """ironcore/layers/mlp.py:19-54 without dropout (inference): a gated
    activation doubles the up-projection (mlp.py:31-33).  Note that the inner
    ``nn.Linear`` of geglu/siglu is built ``d_model`` wide in the reference
    (mlp.py:26-28) while it is applied to ``d_ffn``-wide halves, so those two
    variants only run when ``d_ffn == d_model``; glu and swiglu have no such
    layer."""

    def __init__(self, config):
        super().__init__(config)
        bias = not config.model.no_bias
        self.activation = get_activation(config.model.activation_type, config.model.d_model)
        d_up = config.model.d_ffn * (2 if isinstance(self.activation, GLUActivation) else 1)
        self.up_proj = Linear(config, config.model.d_model, d_up, bias)
        self.down_proj = Linear(config, config.model.d_ffn, config.model.d_model, bias)

    def forward(self, x):
        return self.down_proj(self.activation(self.up_proj(x)))


class TransformerLayer(BaseModule):
    """ironcore/models/transformer.py:23-135.  The new K/V rows exist right
    after the projections (transformer.py:88-98): that is where they enter the
    cache, inside ``self_attention``."""

    def __init__(self, config):
        super().__init__(config)
        m = config.model
        bias = not m.no_bias
        self.head_dimension = m.d_model // m.num_attention_heads
        self.num_local_attention_heads = m.num_attention_heads // config.trainer.tensor_model_parallel_size
        self.num_local_attention_groups = m.num_attention_groups // config.trainer.tensor_model_parallel_size
        self.linear_q = Linear(config, m.d_model, m.head_dim * m.num_attention_heads, bias)
        self.linear_kv = Linear(config, m.d_model, m.head_dim * m.num_attention_groups * 2, bias)
        self.attn_output = Linear(config, m.head_dim * m.num_attention_heads, m.d_model, bias)
        self.input_layernorm = get_layernorm(config)
        self.self_attention = Attention(config)
        self.post_attn_layernorm = get_layernorm(config)
        self.mlp = MLP(config)

    def forward(self, hidden_states, attention_mask, rotary_pos_emb=None, *, kv_cache=None,
                attn_metadata=None):
        b, s, _ = hidden_states.shape
        norm_output = self.input_layernorm(hidden_states)
        query = self.linear_q(norm_output)
        key, value = torch.chunk(self.linear_kv(norm_output), 2, dim=-1)
        query = query.view(b, s, self.num_local_attention_heads, self.head_dimension)
        key = key.view(b, s, self.num_local_attention_groups, self.head_dimension)
        value = value.view(b, s, self.num_local_attention_groups, self.head_dimension)
        # transformer.py:95-98.  Without a cache the rows are rotated here, at
        # their index in the sequence; with a cache the rotation is fused into
        # the KV append inside the attention call.
        if rotary_pos_emb is not None and kv_cache is None:
            positions = torch.arange(s, device=query.device, dtype=torch.int32).repeat(b)
            query = rotary_pos_emb(query, positions)
            key = rotary_pos_emb(key, positions)
        attention_output = self.self_attention(query, key, value, attention_mask, kv_cache=kv_cache,
                                               attn_metadata=attn_metadata,
                                               rotary_pos_emb=rotary_pos_emb if kv_cache is not None else None)
        attention_output = self.attn_output(attention_output)
        residual = norm_output if self.config.model.post_ln else hidden_states
        norm_input = residual + attention_output
        norm_output = self.post_attn_layernorm(norm_input)
        mlp_output = self.mlp(norm_output)
        residual = norm_output if self.config.model.post_ln else norm_input
        return residual + mlp_output


class TransformerModel(BaseModule):
    """ironcore/models/transformer.py:138-162."""

    def __init__(self, config):
        super().__init__(config)
        self.layers = nn.ModuleList([TransformerLayer(config) for _ in range(config.model.num_layers)])

    def forward(self, hidden_states, attention_mask, rotary_pos_emb=None, *, kv_cache: Optional[PagedKVCache] = None,
                attn_metadata=None):
        for index, layer in enumerate(self.layers):
            hidden_states = layer(hidden_states, attention_mask, rotary_pos_emb,
                                  kv_cache=None if kv_cache is None else kv_cache.layer(index),
                                  attn_metadata=attn_metadata)
        return hidden_states


class LanguageModelEmbedding(BaseModule):
    """ironcore/layers/embedding.py:9-50 (word + learned absolute position)."""

    def __init__(self, config, padded_vocab_size: int):
        super().__init__(config)
        kind = config.model.positional_embedding.type
        if kind not in ("absolute", "rope", "none"):
            raise ValueError(f"unknown positional embedding type {kind!r}")
        self.word_embeddings = nn.Embedding(padded_vocab_size, config.model.d_model)
        self.position_embedding = None
        if kind == "absolute":  # embedding.py:16
            self.position_embedding = nn.Embedding(config.model.max_seq_len, config.model.d_model)

    def forward(self, input_ids, position_ids):
        x = self.word_embeddings(input_ids)
        if self.position_embedding is not None:
            x = x + self.position_embedding(position_ids)
        return x


def padded_vocab(vocab_size: int, unit: int = 128) -> int:
    """The reference pads the vocabulary to a multiple of 128 and zeroes the
    padded rows (ironcore/tokenizer/tokenizer.py:70-75,
    ironcore/parallel/tensor_parallel/layers.py:116-118)."""
    return (vocab_size + unit - 1) // unit * unit


class LanguageModel(BaseModule):
    """ironcore/language_model.py:21-100,203-227, inference only (labels=None):
    returns logits ``[b, s, padded_vocab]``.

    ``forward(input_ids)`` is the reference's full causal pass.
    ``forward(input_ids, kv_cache=cache, seq_ids=ids)`` treats ``input_ids`` as
    the NEW tokens of sequences that already live in ``cache`` (prefill when
    they are empty, one token per step afterwards)."""

    def __init__(self, config, vocab_size: int = 50257):
        super().__init__(config)
        self.vocab_size = vocab_size
        self.padded_vocab_size = padded_vocab(vocab_size, config.trainer.vocab_padding_unit)
        self.embedding = LanguageModelEmbedding(config, self.padded_vocab_size)
        self.rotary_pos_emb = None
        if config.model.positional_embedding.type == "rope":  # language_model.py:39-47
            pe = config.model.positional_embedding
            self.rotary_pos_emb = RotaryPositionalEmbedding(
                config.model.d_model // config.model.num_attention_heads, config.model.max_position_embeddings,
                base=pe.base, scale=pe.scaling_factor, offset=pe.offset)
        self.model = TransformerModel(config)
        self.output_layernorm = get_layernorm(config)
        if config.model.untie_embed:
            self.output_layer = Linear(config, config.model.d_model, self.padded_vocab_size, bias=False)
        self.init_weights()

    def init_weights(self):
        """The layers' initialisation (ironcore/layers/module.py:43-76), then the
        padded vocabulary rows zeroed."""
        super().init_weights()
        with torch.no_grad():
            self.embedding.word_embeddings.weight[self.vocab_size:].zero_()

    def forward(self, input_ids, labels=None, *, kv_cache: Optional[PagedKVCache] = None,
                seq_ids: Optional[Sequence[int]] = None, attn_metadata=None, position_ids=None,
                new_token_counts: Optional[Sequence[int]] = None):
        if labels is not None:
            raise NotImplementedError("loss computation is a training feature")
        b, s = input_ids.shape
        dev = input_ids.device
        if attn_metadata is not None:
            # the caller did the cache bookkeeping itself (device-side, for a captured decode step)
            if kv_cache is None or position_ids is None:
                raise ValueError("attn_metadata comes with kv_cache and position_ids")
            meta, attention_mask = attn_metadata, None
        elif kv_cache is None:
            attention_mask = torch.tril(torch.ones(s, s, device=dev)).view(1, 1, s, s) > 0.5
            position_ids = torch.arange(s, device=dev).unsqueeze(0).expand(b, s)
            meta = None
        else:
            if seq_ids is None or len(seq_ids) != b:
                raise ValueError("one cache sequence id per batch row")
            past = [kv_cache.length(sid) for sid in seq_ids]
            # new_token_counts: row i of input_ids holds that many new tokens, the rest is padding
            meta = kv_cache.prepare(seq_ids, s if new_token_counts is None else list(new_token_counts))
            attention_mask = None
            position_ids = (torch.tensor(past, device=dev).unsqueeze(1) + torch.arange(s, device=dev).unsqueeze(0))
        x = self.embedding(input_ids, position_ids)
        x = self.model(x, attention_mask, self.rotary_pos_emb, kv_cache=kv_cache, attn_metadata=meta)
        x = self.output_layernorm(x)
        if self.config.model.untie_embed:
            return torch.matmul(x, self.output_layer.weight)
        return torch.matmul(x, self.embedding.word_embeddings.weight.transpose(0, 1))


def sample_next(logits: torch.Tensor, temperature: float = 0.0, top_k: int = 0,
                generator: Optional[torch.Generator] = None) -> torch.Tensor:
    """Next token from last-position logits ``[b, vocab]``.  ``temperature == 0``
    is greedy argmax; otherwise temperature and top-k sampling exactly as
    examples/generate_text.py:28-37 does them (scale, drop everything below the
    k-th logit, softmax, multinomial)."""
    if temperature == 0.0:
        return logits.argmax(dim=-1, keepdim=True)
    logits = logits / temperature
    if top_k > 0:
        kth = torch.topk(logits, top_k)[0][..., -1, None]
        logits = logits.masked_fill(logits < kth, float("-inf"))
    probs = torch.softmax(logits, dim=-1)
    return torch.multinomial(probs, num_samples=1, generator=generator)


@torch.no_grad()
def generate(model: LanguageModel, input_ids: torch.Tensor, max_new_tokens: int, *,
             block_size: int = 16, temperature: float = 0.0, top_k: int = 0,
             eos_token_id: Optional[int] = None, generator: Optional[torch.Generator] = None,
             kv_cache: Optional[PagedKVCache] = None, return_margins: bool = False,
             use_graph: bool = False, prompt_lens: Optional[Sequence[int]] = None):
    """Batched generation through the block KV cache: one prefill pass over the
    prompts, then one cached decode step per new token.  Prompts ``[b, s]``;
    returns ``[b, s + n]`` token ids (and, on request, the per-step top-1/top-2
    logit margins ``[b, n]``).  The next token is always chosen from the last
    position's logits, as examples/generate_text.py:27-28 does.

    ``prompt_lens``: prompts of unequal length, row i of ``input_ids`` holding
    ``prompt_lens[i]`` tokens and then padding; they are prefilled in one step
    and the result is a list of 1-D tensors, each prompt with its continuation.

    ``use_graph`` (greedy only) captures one decode step, cache bookkeeping and
    token selection included, into a HIP graph and replays it: same tokens,
    without the per-step launch and host work that bounds small models."""
    model.eval()
    b, s = input_ids.shape
    cfg = model.config.model
    if s + max_new_tokens > cfg.max_seq_len:
        raise ValueError("prompt + new tokens exceed the position table")
    if prompt_lens is not None:
        prompt_lens = [int(n) for n in prompt_lens]
        if len(prompt_lens) != b or min(prompt_lens) < 1 or max(prompt_lens) > s:
            raise ValueError("one prompt length in [1, s] per row of input_ids")
    if use_graph:
        if temperature != 0.0:
            raise ValueError("use_graph selects tokens greedily (temperature 0)")
        return _generate_graphed(model, input_ids, max_new_tokens, block_size, eos_token_id, kv_cache,
                                 return_margins, prompt_lens)
    own_cache = kv_cache is None
    if own_cache:
        per_seq = (s + max_new_tokens + block_size - 1) // block_size
        kv_cache = PagedKVCache(cfg.num_layers, b * per_seq, block_size, cfg.num_attention_groups,
                                cfg.d_model // cfg.num_attention_heads,
                                next(model.parameters()).dtype, input_ids.device)
    seq_ids = [kv_cache.add_sequence() for _ in range(b)]
    tokens = input_ids
    margins = []
    finished = torch.zeros(b, dtype=torch.bool, device=input_ids.device)
    step_input = input_ids
    for step in range(max_new_tokens):
        if step == 0:
            logits = _prefill_logits(model, input_ids, prompt_lens, kv_cache, seq_ids)
        else:
            logits = model(step_input, kv_cache=kv_cache, seq_ids=seq_ids)[:, -1, :]
        if return_margins:
            top2 = torch.topk(logits.float(), 2, dim=-1)[0]
            margins.append(top2[:, 0] - top2[:, 1])
        nxt = sample_next(logits, temperature, top_k, generator)
        if eos_token_id is not None:
            nxt = torch.where(finished.unsqueeze(1), torch.full_like(nxt, eos_token_id), nxt)
            finished |= nxt.squeeze(1) == eos_token_id
        tokens = torch.cat([tokens, nxt], dim=1)
        step_input = nxt
        if eos_token_id is not None and bool(finished.all()):
            break
    if own_cache:
        for sid in seq_ids:
            kv_cache.free_sequence(sid)
    tokens = _with_prompts(tokens, s, prompt_lens)
    if return_margins:
        return tokens, torch.stack(margins, dim=1)
    return tokens


def _prefill_logits(model, input_ids, prompt_lens, kv_cache, seq_ids):
    """Logits ``[b, vocab]`` at each prompt's last token after one prefill step."""
    if prompt_lens is None:
        return model(input_ids, kv_cache=kv_cache, seq_ids=seq_ids)[:, -1, :]
    logits = model(input_ids, kv_cache=kv_cache, seq_ids=seq_ids, new_token_counts=prompt_lens)
    last = torch.tensor(prompt_lens, device=input_ids.device) - 1
    return logits[torch.arange(len(prompt_lens), device=input_ids.device), last]


def _with_prompts(tokens, s, prompt_lens):
    """``tokens`` is [b, s + n] with the new tokens behind the padded prompts:
    with prompts of unequal length, a list of prompt + continuation per row."""
    if prompt_lens is None:
        return tokens
    return [torch.cat([row[:n], row[s:]]) for row, n in zip(tokens, prompt_lens)]


def _generate_graphed(model, input_ids, max_new_tokens, block_size, eos_token_id, kv_cache, return_margins,
                      prompt_lens=None):
    """The loop of :func:`generate` with everything a decode step needs kept on
    the device: the sequences' blocks are reserved up front, the step derives
    the new token's position and pool slot from the context lengths it
    increments itself, and writes the chosen token into column ``col`` of the
    output.  The prefill and the first decode step run eagerly (the second
    also serves as the warm-up a capture needs); the rest are replays."""
    b, s = input_ids.shape
    dev = input_ids.device
    cfg = model.config.model
    if max_new_tokens < 1:
        return (input_ids, input_ids.new_zeros(b, 0, dtype=torch.float32)) if return_margins else input_ids
    own_cache = kv_cache is None
    if own_cache:
        per_seq = (s + max_new_tokens + block_size - 1) // block_size
        kv_cache = PagedKVCache(cfg.num_layers, b * per_seq, block_size, cfg.num_attention_groups,
                                cfg.d_model // cfg.num_attention_heads,
                                next(model.parameters()).dtype, dev)
    bs = kv_cache.block_size
    seq_ids = [kv_cache.add_sequence() for _ in range(b)]
    logits = _prefill_logits(model, input_ids, prompt_lens, kv_cache, seq_ids)

    # the last token chosen is never fed back
    cached_at_end = max(kv_cache.length(sid) for sid in seq_ids) + max_new_tokens - 1
    for sid in seq_ids:
        kv_cache.reserve(sid, kv_cache.length(sid) + max_new_tokens - 1)
    tables = kv_cache.block_table(seq_ids)
    ctx = torch.tensor([kv_cache.length(sid) for sid in seq_ids], dtype=torch.int32, device=dev)
    new_tokens = torch.zeros(b, max_new_tokens, dtype=torch.int64, device=dev)
    margins = torch.zeros(b, max_new_tokens, dtype=torch.float32, device=dev) if return_margins else None
    col = torch.zeros(1, 1, dtype=torch.int64, device=dev)
    step_input = torch.zeros(b, 1, dtype=torch.int64, device=dev)
    finished = torch.zeros(b, dtype=torch.bool, device=dev)

    def select(logits):
        if margins is not None:
            top2 = torch.topk(logits.float(), 2, dim=-1)[0]
            margins.scatter_(1, col.expand(b, 1), (top2[:, 0] - top2[:, 1]).unsqueeze(1))
        nxt = logits.argmax(dim=-1, keepdim=True)
        if eos_token_id is not None:
            nxt = torch.where(finished.unsqueeze(1), torch.full_like(nxt, eos_token_id), nxt)
            finished.logical_or_(nxt.squeeze(1) == eos_token_id)
        new_tokens.scatter_(1, col.expand(b, 1), nxt)
        col.add_(1)
        step_input.copy_(nxt)

    def decode_step():
        pos = ctx.clone()                                    # the new token's position = tokens cached so far
        ctx.add_(1)
        block = tables.gather(1, (pos // bs).long().unsqueeze(1)).squeeze(1)
        meta = PagedAttentionMetadata(
            block_tables=tables, context_lens=ctx, slot_mapping=block.long() * bs + (pos % bs).long(),
            max_context_len=cached_at_end, cu_seqlens_q=None, cohort_size=1, cohort_shared_blocks=None,
            positions=pos)
        step_logits = model(step_input, kv_cache=kv_cache, attn_metadata=meta,
                            position_ids=pos.long().unsqueeze(1))[:, -1, :]
        select(step_logits)

    select(logits)
    steps_run = 0
    if max_new_tokens > 1:
        decode_step()
        steps_run = 1
    if max_new_tokens > 2:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            decode_step()
        for i in range(max_new_tokens - 2):
            graph.replay()
            steps_run += 1
            if eos_token_id is not None and i % 8 == 7 and bool(finished.all()):
                break
    kv_cache.advance(seq_ids, steps_run)
    n = steps_run + 1
    if eos_token_id is not None:
        # what the step-by-step loop returns: it stops right after the step at which every row has ended
        ended = ((new_tokens[:, :n] == eos_token_id).cumsum(1) > 0).all(0)
        if bool(ended.any()):
            n = int(ended.int().argmax()) + 1
    tokens = _with_prompts(torch.cat([input_ids, new_tokens[:, :n]], dim=1), s, prompt_lens)
    if own_cache:
        for sid in seq_ids:
            kv_cache.free_sequence(sid)
    if return_margins:
        return tokens, margins[:, :n]
    return tokens


@torch.no_grad()
def generate_samples(model: LanguageModel, prompt_ids: torch.Tensor, n_samples: int, max_new_tokens: int, *,
                     block_size: int = 16, temperature: float = 1.0, top_k: int = 0,
                     generator: Optional[torch.Generator] = None, kv_cache: Optional[PagedKVCache] = None):
    """``n_samples`` continuations of every prompt (rollouts of one policy on
    one prompt, as GRPO-style training draws them).  Each prompt ``[p, s]`` is
    prefilled ONCE; its samples are forks of that sequence, so they alias the
    prompt's full blocks in the pools, and every decode step runs them as
    cohorts: the shared blocks are streamed once per cohort, not once per
    sample.  Returns ``[p, n_samples, s + n]`` token ids.  Token selection is
    :func:`sample_next` (examples/generate_text.py:28-37); temperature 0 gives
    ``n_samples`` copies of the greedy continuation."""
    model.eval()
    p, s = prompt_ids.shape
    cfg = model.config.model
    if s + max_new_tokens > cfg.max_seq_len:
        raise ValueError("prompt + new tokens exceed the position table")
    dev = prompt_ids.device
    own_cache = kv_cache is None
    if own_cache:
        shared = s // block_size
        own = (s + max_new_tokens + block_size - 1) // block_size - shared
        kv_cache = PagedKVCache(cfg.num_layers, p * (shared + n_samples * own), block_size,
                                cfg.num_attention_groups, cfg.d_model // cfg.num_attention_heads,
                                next(model.parameters()).dtype, dev)
    roots = [kv_cache.add_sequence() for _ in range(p)]
    logits = model(prompt_ids, kv_cache=kv_cache, seq_ids=roots)[:, -1, :]
    seq_ids = []
    for root in roots:                        # the samples of a prompt side by side: one cohort each
        seq_ids += [root] + [kv_cache.fork(root) for _ in range(n_samples - 1)]
    logits = logits.repeat_interleave(n_samples, dim=0)
    group = cfg.num_attention_heads // cfg.num_attention_groups
    fits = group <= 16 and n_samples <= 8 * (16 // group) and next(model.parameters()).dtype != torch.float32
    tokens = prompt_ids.repeat_interleave(n_samples, dim=0)
    for step in range(max_new_tokens):
        if step:
            meta = kv_cache.prepare(seq_ids, 1, cohort_size=n_samples if fits else 1)
            past = torch.tensor([kv_cache.length(sid) - 1 for sid in seq_ids], device=dev).unsqueeze(1)
            logits = model(nxt, kv_cache=kv_cache, attn_metadata=meta, position_ids=past)[:, -1, :]
        nxt = sample_next(logits, temperature, top_k, generator)
        tokens = torch.cat([tokens, nxt], dim=1)
    if own_cache:
        for sid in seq_ids:
            kv_cache.free_sequence(sid)
    return tokens.view(p, n_samples, s + max_new_tokens)


@torch.no_grad()
def generate_full_recompute(model: LanguageModel, input_ids: torch.Tensor, max_new_tokens: int):
    """The reference's loop (examples/generate_text.py:24-40) with greedy
    selection: the whole sequence goes through the model at every step."""
    model.eval()
    tokens = input_ids
    for _ in range(max_new_tokens):
        logits = model(tokens)[:, -1, :]
        tokens = torch.cat([tokens, logits.argmax(dim=-1, keepdim=True)], dim=1)
    return tokens
