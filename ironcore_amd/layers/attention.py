"""Attention layer: the reference's call signature, MI355X kernels underneath.

Mirror of ``ironcore.layers.attention.Attention``
(ironcore/layers/attention.py:24-253): same constructor argument, same
attributes (attention.py:44-66), same ``forward(query, key, value,
attention_mask=None)`` with ``query [b, sq, hn, hd]``, ``key``/``value``
``[b, sk, gn, hd]`` and result ``[b, sq, hn*hd]`` (attention.py:208-253), same
GQA head map (query head h reads KV head h // (hn // gn), attention.py:95-102)
and the same scale 1/sqrt(d_model // hn) (attention.py:51,65,110).

The block-KV-cache path is reached only through the two extra keyword
arguments, so the reference's call site
(ironcore/models/transformer.py:101-103) stays valid unchanged:

    attn(query, key, value, attention_mask, kv_cache=layer_cache, attn_metadata=meta)

appends the new ``key``/``value`` rows to the layer's block pool and attends
against the cache (decode kernel for sq == 1, chunked-prefill kernel
otherwise).  Without ``kv_cache`` the call is the reference's dense call; it
runs on the same chunked-prefill kernel by viewing ``key``/``value`` as a pool
with one block per sequence.  bf16 and fp16 tensors take the 16-bit matrix-core
kernels, fp32 tensors (what the reference's own contract tests pass,
tests/test_attention.py:143-161) the fp32 ones, with every product, sum and
probability in fp32.  The reference's second branch is kept as well: when
``config.trainer.use_flash_attn`` is set and the flash-attn import worked, the
dense call goes through ``_flash_attention`` (causal, the mask ignored,
attention.py:230-250), here on the same kernels.  Every path runs the
hand-written HIP kernels; there is no torch fallback.
"""
from __future__ import annotations

import weakref
from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn.functional as F
from torch import nn

from .. import paged_ops
from .module import BaseModule, get_model_dtype

# The reference takes its flash branch only when this import worked
# (ironcore/layers/attention.py:14-17,230).  Here the name is nothing but that
# switch: the branch runs on the kernels of this package, never on the wheel.
try:
    from flash_attn import flash_attn_varlen_func
except ImportError:
    flash_attn_varlen_func = None


# attention_mask tensor -> what _classify_mask found for it: id -> (weak reference, (version, shapes), kind, bytes).
# An entry goes when its mask tensor dies (the weak reference's callback) and when more than
# _MASK_CLASSES_MAX masks are alive at once (oldest first): the byte copy of a general mask is as
# large as the mask, and a model that builds a new document mask per batch must not pile them up.
_MASK_CLASSES: dict = {}
_MASK_CLASSES_MAX = 4


def _mask_version(mask):
    """The tensor's in-place edit counter, or None for a tensor that keeps none
    (one created under torch.inference_mode()): such a mask is classified on
    every call, since an edit to it could not be noticed."""
    try:
        return mask._version
    except RuntimeError:
        return None


@dataclass
class PagedAttentionMetadata:
    """What one forward pass over a batch needs to know about the block KV
    cache (built by ``ironcore_amd.kv_cache.PagedKVCache.prepare``).

    block_tables   int32 [b, max_blocks]   pool block of each sequence block
    context_lens   int32 [b]               tokens visible after this step's append
    slot_mapping   int64 [b*sq]            pool slot of every new token, row-major
                                           over (sequence, position); -1 = padding
    max_context_len  host-side upper bound on context_lens
    positions      int32 [b*sq]            index of every new token in its sequence
                                           (the rotary table row; 0 for padding)
    cohort_size, cohort_shared_blocks
                   optional: consecutive groups of ``cohort_size`` sequences
                   whose first ``cohort_shared_blocks[i]`` table entries are the
                   same pool blocks (forked prompts); decode then reads those
                   blocks once per cohort
    """
    block_tables: torch.Tensor
    context_lens: torch.Tensor
    slot_mapping: torch.Tensor
    max_context_len: int
    cu_seqlens_q: Optional[torch.Tensor] = None   # int32 [b+1]; built on demand for prefill
    cohort_size: int = 1
    cohort_shared_blocks: Optional[torch.Tensor] = None   # int32 [ceil(b / cohort_size)]
    positions: Optional[torch.Tensor] = None   # int32 [b*sq]: index of every new token in its sequence
    # Chunks of unequal length in one step: cu_seqlens_q holds the true bounds,
    # chunk_rows (int64 [sum of chunk lengths]) the rows of the padded [b*sq]
    # layout that exist, max_chunk_len the longest chunk.
    chunk_rows: Optional[torch.Tensor] = None
    max_chunk_len: int = 0


class Attention(BaseModule):
    """Attention math only (no projections), as in the reference."""

    def __init__(self, config):
        super().__init__(config)
        self.num_attention_heads = config.model.num_attention_heads
        self.tensor_model_parallel_size = config.trainer.tensor_model_parallel_size
        self.head_dimension = config.model.d_model // self.num_attention_heads
        self.num_local_attention_heads = self.num_attention_heads // self.tensor_model_parallel_size
        self.num_local_attention_groups = (
            config.model.num_attention_groups // self.tensor_model_parallel_size)
        self.softmax = torch.nn.Softmax(dim=-1)
        self.attn_dropout = nn.Dropout(config.model.dropout_attn)
        self.scale_factor = self.head_dimension ** 0.5
        self.mask_value = torch.finfo(get_model_dtype(config)).min

    # ------------------------------------------------------------------ helpers
    def _check_shapes(self, query, key, value):
        if query.dim() != 4 or key.dim() != 4 or value.shape != key.shape:
            raise ValueError("expected query [b, sq, hn, hd] and key/value [b, sk, gn, hd]")
        b, sq, hn, hd = query.shape
        if hn != self.num_local_attention_heads or key.shape[2] != self.num_local_attention_groups:
            raise ValueError(
                f"got {hn} query / {key.shape[2]} KV heads, layer has "
                f"{self.num_local_attention_heads} / {self.num_local_attention_groups}")
        if hd != self.head_dimension or key.shape[3] != hd:
            raise ValueError(f"head dimension {hd} != d_model // heads = {self.head_dimension}")
        if self.training and self.config.model.dropout_attn > 0.0:
            raise NotImplementedError("attention dropout is a training feature; the paged "
                                      "kernels implement the inference path (dropout_attn == 0 or eval())")
        if torch.is_grad_enabled() and (query.requires_grad or key.requires_grad or value.requires_grad):
            # The reference's layer is differentiable (its tests backpropagate through it,
            # tests/test_attention.py:391-426); the HIP kernels are forward only and their output
            # carries no graph, so a backward pass would silently leave attention and the Q/K/V
            # projections without gradient.
            raise NotImplementedError(
                "the HIP attention path is forward only: query/key/value require grad and autograd is "
                "recording; call it under torch.no_grad() / torch.inference_mode() or on detached tensors")

    def _classify_mask(self, attention_mask, b, sq, sk, hn):
        """What the kernels have to do for this mask (0 = hidden, broadcastable
        to [b, hn, sq, sk], attention.py:115-117): ``("none", None)`` when every
        key is visible, ``("causal", None)`` for the lower-triangular pattern the
        reference model builds (ironcore/language_model.py:109-114,159; shifted
        when sq < sk), else ``("general", bytes)`` with the mask as a uint8
        ``[1 or b, 1 or hn, sq, sk]`` tensor for the masked kernels.

        Telling the patterns apart needs a look at the values (one device
        synchronisation); the answer is remembered per mask TENSOR (identity
        and version counter), so a model that hands one mask to all its layers
        pays once per forward pass, not once per layer."""
        if attention_mask is None:
            return "none", None
        version = _mask_version(attention_mask)
        hit = _MASK_CLASSES.get(id(attention_mask)) if version is not None else None
        if hit is not None and hit[0]() is attention_mask and hit[1] == (version, b, sq, sk, hn):
            return hit[2], hit[3]
        m = attention_mask
        while m.dim() < 4:
            m = m.unsqueeze(0)
        if m.dim() != 4 or m.shape[-2:] != (sq, sk) or m.shape[0] not in (1, b) or m.shape[1] not in (1, hn):
            raise ValueError(f"attention_mask must be broadcastable to [{b}, {hn}, {sq}, {sk}], "
                             f"got {tuple(attention_mask.shape)}")
        visible = m != 0
        i = torch.arange(sq, device=m.device).unsqueeze(1)
        j = torch.arange(sk, device=m.device).unsqueeze(0)
        want = j <= (sk - sq) + i
        flags = torch.stack([visible.all(), (visible == want).all()]).tolist()   # the one synchronisation
        if flags[0]:
            kind, data = "none", None
        elif flags[1] and sq <= sk:
            kind, data = "causal", None
        else:
            kind, data = "general", visible.to(torch.uint8).contiguous()
        if version is not None:
            key = id(attention_mask)
            _MASK_CLASSES.pop(key, None)
            while len(_MASK_CLASSES) >= _MASK_CLASSES_MAX:
                del _MASK_CLASSES[next(iter(_MASK_CLASSES))]

            def forget(ref, key=key):
                if key in _MASK_CLASSES and _MASK_CLASSES[key][0] is ref:
                    del _MASK_CLASSES[key]
            _MASK_CLASSES[key] = (weakref.ref(attention_mask, forget), (version, b, sq, sk, hn), kind, data)
        return kind, data

    # ------------------------------------------------------------------ forward
    def forward(self, query, key, value, attention_mask=None, *, kv_cache=None, attn_metadata=None,
                rotary_pos_emb=None):
        """query [b, sq, hn, hd]; key/value [b, sk, gn, hd]; returns [b, sq, hn*hd].

        ``rotary_pos_emb`` (cached path only): a rotary module whose rotation
        of query and key has NOT been applied yet; it is fused into the KV
        append, at the positions ``attn_metadata.positions`` names."""
        self._check_shapes(query, key, value)
        if kv_cache is not None:
            return self._paged(query, key, value, kv_cache, attn_metadata, rotary_pos_emb)
        if rotary_pos_emb is not None:
            raise ValueError("without a KV cache, rotate query and key before the call "
                             "(ironcore/models/transformer.py:95-98)")
        if self.config.trainer.use_flash_attn and flash_attn_varlen_func is not None:
            # the reference's flash branch: causal, the mask ignored (attention.py:230,240-250)
            sq, sk = query.size(1), key.size(1)
            return self._flash_attention(query, key, value, sq, sk, sq, sk, causal=True, window_size=(-1, -1))
        return self._dense(query, key, value, attention_mask)

    def _flash_attention(self, query, key, value, seq_len_q, seq_len_kv, max_seqlen_q, max_seqlen_k,
                         causal=False, window_size=(-1, -1), alibi_slopes=None):
        """The reference's flash branch (attention.py:144-206) on this package's
        kernels: every sequence whole (the reference builds equal-length
        cu_seqlens, attention.py:170-183), ``causal`` aligned to the bottom
        right as flash-attn aligns it (row i sees keys j <= (sk - sq) + i; a row
        that sees no key returns zeros), which for sq == sk is the mask the
        reference's own tests set beside it (tests/test_attention.py:618-671).
        KV heads follow the GQA map of the dense branch, as those tests expect
        (:673-730).  Sliding windows, ALiBi slopes and attention dropout (which
        the wheel applies whatever the module's mode) are not built."""
        if tuple(window_size) != (-1, -1) or alibi_slopes is not None:
            raise NotImplementedError("sliding-window and ALiBi attention are not built")
        if self.config.model.dropout_attn > 0.0:
            raise NotImplementedError("the flash branch applies dropout_attn in every mode; the kernels "
                                      "implement dropout_attn == 0")
        b, sq, hn, hd = query.shape
        sk = key.shape[1]
        if (seq_len_q, seq_len_kv) != (sq, sk):
            raise ValueError(f"seq_len_q / seq_len_kv {seq_len_q} / {seq_len_kv} do not match the tensors ({sq} / {sk})")
        if not causal or sq <= sk:
            return self._attend_dense(query, key, value, bool(causal), None)
        out = query.new_zeros(b, sq, hn * hd)   # rows above the bottom-right triangle see no key
        if sk > 0:
            out[:, sq - sk:] = self._attend_dense(query[:, sq - sk:], key, value, True, None)
        return out

    def _dense(self, query, key, value, attention_mask):
        b, sq, hn, hd = query.shape
        sk = key.shape[1]
        kind, mask = self._classify_mask(attention_mask, b, sq, sk, hn)
        return self._attend_dense(query, key, value, kind == "causal", mask)

    def _attend_dense(self, query, key, value, causal, mask):
        b, sq, hn, hd = query.shape
        if hd not in paged_ops.SUPPORTED_HEAD_DIMS:
            # The reference takes any d_model // heads (attention.py:51).  Zero columns appended
            # to query, key and value change no score (the scale stays 1/sqrt(hd)) and add zero
            # output columns, so a head dimension between the built ones runs on the next one up.
            wide = next((w for w in paged_ops.SUPPORTED_HEAD_DIMS if w > hd), None)
            if wide is None:
                raise ValueError(f"head dimension {hd}: the attention kernels are built for "
                                 f"{paged_ops.SUPPORTED_HEAD_DIMS} and pad smaller ones up to the next of them")
            pad = (0, wide - hd)
            padded = self._dense_on_kernel_width(F.pad(query, pad), F.pad(key, pad), F.pad(value, pad), causal, mask)
            return padded.view(b, sq, hn, wide)[..., :hd].reshape(b, sq, hn * hd)
        return self._dense_on_kernel_width(query, key, value, causal, mask)

    def _dense_on_kernel_width(self, query, key, value, causal, mask):
        b, sq, hn, hd = query.shape
        sk, gn = key.shape[1], key.shape[2]
        key, value = key.contiguous(), value.contiguous()
        # one pool block per sequence: [b, gn, sk, hd] view of the [b, sk, gn, hd] rows
        k_pool, v_pool = key.permute(0, 2, 1, 3), value.permute(0, 2, 1, 3)
        dev = query.device
        tables = torch.arange(b, dtype=torch.int32, device=dev).unsqueeze(1)
        ctx = torch.full((b,), sk, dtype=torch.int32, device=dev)
        cu = torch.arange(0, (b + 1) * sq, sq, dtype=torch.int32, device=dev)
        out = paged_ops.paged_prefill(query.reshape(b * sq, hn, hd), k_pool, v_pool, tables, ctx, cu, sq,
                                      causal=causal, scale=1.0 / self.scale_factor, mask=mask)
        return out.view(b, sq, hn * hd)

    def _ragged_chunks(self, query, k_pool, v_pool, meta, rows, scale):
        """Chunks of unequal length, padded to [b, sq]: the rows that exist are
        packed for the kernel and its output rows put back; padding rows
        return zeros."""
        b, sq, hn, hd = query.shape
        packed = query.reshape(b * sq, hn, hd).index_select(0, rows)
        got = paged_ops.paged_prefill(packed, k_pool, v_pool, meta.block_tables, meta.context_lens,
                                      meta.cu_seqlens_q, meta.max_chunk_len, causal=True, scale=scale)
        out = query.new_zeros(b * sq, hn * hd)
        out.index_copy_(0, rows, got)
        return out.view(b, sq, hn * hd)

    def _paged(self, query, key, value, kv_cache, meta, rotary_pos_emb=None):
        if meta is None:
            raise ValueError("kv_cache needs attn_metadata")
        b, sq, hn, hd = query.shape
        gn = key.shape[2]
        if key.shape[1] != sq:
            raise ValueError("with a KV cache, key/value carry only the new tokens (sk == sq)")
        k_pool, v_pool = kv_cache
        if rotary_pos_emb is None:
            paged_ops.kv_append(key.reshape(b * sq, gn, hd), value.reshape(b * sq, gn, hd), k_pool, v_pool,
                                meta.slot_mapping)
        else:
            if meta.positions is None:
                raise ValueError("rotary embeddings in the cached path need attn_metadata.positions")
            rotated = query.reshape(b * sq, hn, hd).clone(memory_format=torch.contiguous_format)
            paged_ops.rope_kv_append(rotated, key.reshape(b * sq, gn, hd), value.reshape(b * sq, gn, hd),
                                     k_pool, v_pool, meta.slot_mapping, meta.positions,
                                     rotary_pos_emb.cos_emb, rotary_pos_emb.sin_emb)
            query = rotated.view(b, sq, hn, hd)
        scale = 1.0 / self.scale_factor
        rows = getattr(meta, "chunk_rows", None)
        if rows is not None:
            return self._ragged_chunks(query, k_pool, v_pool, meta, rows, scale)
        if sq == 1:
            cohort = meta.cohort_size if query.dtype != torch.float32 else 1
            out = paged_ops.paged_decode(query.view(b, hn, hd), k_pool, v_pool, meta.block_tables,
                                         meta.context_lens, meta.max_context_len, scale=scale,
                                         cohort_size=cohort,
                                         cohort_shared_blocks=meta.cohort_shared_blocks if cohort > 1 else None)
            return out.view(b, 1, hn * hd)
        cu = meta.cu_seqlens_q
        if cu is None:
            cu = torch.arange(0, (b + 1) * sq, sq, dtype=torch.int32, device=query.device)
        out = paged_ops.paged_prefill(query.reshape(b * sq, hn, hd), k_pool, v_pool, meta.block_tables,
                                      meta.context_lens, cu, sq, causal=True, scale=scale)
        return out.view(b, sq, hn * hd)
