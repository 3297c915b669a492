"""Tensor-level wrappers over the C ABI: shape checks, strides, stream.

Every function here runs the hand-written HIP kernels on the tensors' GPU, on
torch's current stream.  CPU tensors are rejected: the paged path has no
non-HIP implementation.

Pool layout: ``k_pool``/``v_pool`` are ``[num_blocks, gn, block_size, hd]``
(any strides with a contiguous last dimension); token ``p`` of sequence ``i``
is ``pool[block_tables[i, p // block_size], :, p % block_size, :]``.
"""
from __future__ import annotations

import math

import torch

from . import _lib


def _require_gpu(*tensors: torch.Tensor) -> torch.device:
    dev = tensors[0].device
    for t in tensors:
        if t.device.type != "cuda":
            raise RuntimeError("paged attention runs on the GPU only (got a tensor on "
                               f"{t.device}); there is no CPU path")
        if t.device != dev:
            raise RuntimeError("all tensors must be on the same device")
    return dev


# Head dimensions the attention kernels are built for (the append kernels take any multiple of
# 16 bytes).  The layer's dense call pads smaller ones up to the next entry.
SUPPORTED_HEAD_DIMS = (32, 64, 128)


def _require_head_dim(hd: int) -> None:
    if hd not in SUPPORTED_HEAD_DIMS:
        raise ValueError(f"the attention kernels are built for head dimensions {SUPPORTED_HEAD_DIMS}, got {hd}")


def _pool_strides(k_pool: torch.Tensor, v_pool: torch.Tensor):
    if k_pool.dim() != 4 or k_pool.shape != v_pool.shape or k_pool.stride() != v_pool.stride():
        raise ValueError("k_pool and v_pool must be [num_blocks, gn, block_size, hd] with equal strides")
    if k_pool.stride(3) != 1:
        raise ValueError("the head dimension of the pools must be contiguous")
    nb, gn, bs, hd = k_pool.shape
    sb, sh, st, _ = k_pool.stride()
    return nb, gn, bs, hd, sb, sh, st


class _Workspace:
    """Split-K scratch, grown on demand, one per (device, stream).  Kernels
    that use it are stream-ordered, so reuse across calls on one stream is
    safe; calls on different streams get different buffers."""

    def __init__(self):
        self._buf: dict[tuple, torch.Tensor] = {}

    def get(self, device: torch.device, nbytes: int) -> torch.Tensor:
        key = (device, _lib.current_stream_ptr(device))
        buf = self._buf.get(key)
        if buf is None or buf.numel() < nbytes:
            buf = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
            self._buf[key] = buf
        return buf


_workspace = _Workspace()


def mfma_probe(iters: int, sink: torch.Tensor) -> int:
    """Launch the matrix-rate probe (``iters`` x 16 register-only
    v_mfma_f32_32x32x16_bf16 per wave, one wave per SIMD on every CU) on the
    current stream and return the launch's flop count.  A diagnostic for the
    benchmark; ``sink`` is any fp32 tensor on the GPU."""
    lib = _lib.load()
    dev = _require_gpu(sink)
    with torch.cuda.device(dev):
        rc = lib.ic_mfma_probe(int(iters), sink.data_ptr(), _lib.current_stream_ptr(dev))
    if rc < 0:
        _lib.check("ic_mfma_probe", int(rc))
    return int(rc)


def kv_append(k_new: torch.Tensor, v_new: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
              slot_mapping: torch.Tensor) -> None:
    """Copy rows ``k_new[t]``, ``v_new[t]`` (``[n, gn, hd]``) into pool slot
    ``slot_mapping[t]`` (= block*block_size + offset), bit for bit.  Negative
    slots are skipped."""
    lib = _lib.load()
    dev = _require_gpu(k_new, v_new, k_pool, v_pool, slot_mapping)
    nb, gn, bs, hd, sb, sh, st = _pool_strides(k_pool, v_pool)
    if k_new.dim() != 3 or k_new.shape != v_new.shape or tuple(k_new.shape[1:]) != (gn, hd):
        raise ValueError(f"k_new/v_new must be [n, {gn}, {hd}], got {tuple(k_new.shape)} / {tuple(v_new.shape)}")
    if k_new.dtype != k_pool.dtype or v_new.dtype != k_pool.dtype:
        raise TypeError("new rows and pools must share a dtype")
    n = k_new.shape[0]
    if slot_mapping.dtype != torch.int64 or slot_mapping.numel() != n or not slot_mapping.is_contiguous():
        raise ValueError("slot_mapping must be a contiguous int64 tensor with one slot per new row")

    def rows_ok(t):
        return t.stride(2) == 1 and t.stride(1) == hd
    if not (rows_ok(k_new) and rows_ok(v_new) and k_new.stride(0) == v_new.stride(0)):
        k_new, v_new = k_new.contiguous(), v_new.contiguous()
    with torch.cuda.device(dev):
        rc = lib.ic_kv_append(k_new.data_ptr(), v_new.data_ptr(), k_new.stride(0),
                              k_pool.data_ptr(), v_pool.data_ptr(), sb, sh, st,
                              slot_mapping.data_ptr(), n, gn, hd, bs, nb,
                              _lib.dtype_code(k_pool.dtype), _lib.current_stream_ptr(dev))
    _lib.check("ic_kv_append", rc)


def rope_kv_append(query: torch.Tensor | None, k_new: torch.Tensor | None, v_new: torch.Tensor | None,
                   k_pool: torch.Tensor | None, v_pool: torch.Tensor | None,
                   slot_mapping: torch.Tensor | None, positions: torch.Tensor,
                   cos_table: torch.Tensor, sin_table: torch.Tensor) -> None:
    """Rotary embedding fused into the append: rotate ``query`` (``[n, hn, hd]``)
    IN PLACE, rotate the rows of ``k_new`` into their pool slots, copy the rows
    of ``v_new`` into theirs.  ``positions`` (int32 ``[n]``) picks each token's
    row of the fp32 ``[rows, hd/2]`` tables.  ``query=None`` skips the query;
    ``k_new=v_new=None`` rotates the query only."""
    lib = _lib.load()
    has_kv = k_new is not None
    tensors = [positions, cos_table, sin_table]
    tensors += [query] if query is not None else []
    tensors += [k_new, v_new, k_pool, v_pool, slot_mapping] if has_kv else []
    dev = _require_gpu(*tensors)
    ref = query if query is not None else k_new
    if ref is None:
        raise ValueError("nothing to do: neither query nor k_new/v_new given")
    n, hd = ref.shape[0], ref.shape[-1]
    if cos_table.dtype != torch.float32 or sin_table.dtype != torch.float32 or cos_table.shape != sin_table.shape \
            or cos_table.dim() != 2 or cos_table.shape[1] != hd // 2 or not cos_table.is_contiguous() \
            or not sin_table.is_contiguous():
        raise ValueError(f"cos_table / sin_table must be contiguous fp32 [rows, {hd // 2}]")
    if positions.dtype != torch.int32 or positions.numel() != n or not positions.is_contiguous():
        raise ValueError("positions must be a contiguous int32 tensor with one entry per token")
    q_ptr, q_stride, hn = 0, 0, 0
    if query is not None:
        if query.dim() != 3 or query.stride(2) != 1 or query.stride(1) != hd:
            raise ValueError("query must be [n, hn, hd] with contiguous heads (it is rotated in place)")
        q_ptr, q_stride, hn = query.data_ptr(), query.stride(0), query.shape[1]
    k_ptr = v_ptr = kp_ptr = vp_ptr = slot_ptr = 0
    new_stride = sb = sh = st = nb = 0
    gn, bs = 1, 16
    if has_kv:
        nb, gn, bs, hd_pool, sb, sh, st = _pool_strides(k_pool, v_pool)
        if hd_pool != hd or k_new.dim() != 3 or k_new.shape != v_new.shape or tuple(k_new.shape) != (n, gn, hd):
            raise ValueError(f"k_new/v_new must be [{n}, {gn}, {hd_pool}]")
        if not (ref.dtype == k_new.dtype == v_new.dtype == k_pool.dtype):
            raise TypeError("query, new rows and pools must share a dtype")
        if slot_mapping.dtype != torch.int64 or slot_mapping.numel() != n or not slot_mapping.is_contiguous():
            raise ValueError("slot_mapping must be a contiguous int64 tensor with one slot per new row")

        def rows_ok(t):
            return t.stride(2) == 1 and t.stride(1) == hd
        if not (rows_ok(k_new) and rows_ok(v_new) and k_new.stride(0) == v_new.stride(0)):
            k_new, v_new = k_new.contiguous(), v_new.contiguous()
        k_ptr, v_ptr, new_stride = k_new.data_ptr(), v_new.data_ptr(), k_new.stride(0)
        kp_ptr, vp_ptr, slot_ptr = k_pool.data_ptr(), v_pool.data_ptr(), slot_mapping.data_ptr()
    with torch.cuda.device(dev):
        rc = lib.ic_rope_kv_append(q_ptr, q_stride, hn, k_ptr, v_ptr, new_stride, kp_ptr, vp_ptr, sb, sh, st,
                                   slot_ptr, positions.data_ptr(), cos_table.data_ptr(), sin_table.data_ptr(),
                                   cos_table.shape[0], n, gn, hd, bs, nb, _lib.dtype_code(ref.dtype),
                                   _lib.current_stream_ptr(dev))
    _lib.check("ic_rope_kv_append", rc)


def paged_decode(query: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                 block_tables: torch.Tensor, context_lens: torch.Tensor, max_context_len: int,
                 scale: float | None = None, out: torch.Tensor | None = None,
                 min_chunk_tokens: int = 0, cohort_size: int = 1,
                 cohort_shared_blocks: torch.Tensor | None = None,
                 key_mask: torch.Tensor | None = None) -> torch.Tensor:
    """One query token per sequence.  ``query`` ``[b, hn, hd]`` -> ``[b, hn*hd]``.

    ``key_mask`` (fp32 only; uint8 ``[b, 1 or hn, >= max_context_len]``,
    contiguous): 0 hides a key from that sequence's query (head); hidden keys
    get the reference's finite fill value, so a query that sees nothing
    averages V over its context.

    ``max_context_len`` is a host-side upper bound on ``context_lens`` (no
    device synchronisation is needed to launch).  ``min_chunk_tokens`` is the
    smallest split-K share (0 = library default).

    Shared prefixes: with ``cohort_size`` S > 1, sequences ``i*S .. i*S+S-1``
    form cohort ``i`` and ``cohort_shared_blocks[i]`` (int32, one per cohort)
    says how many leading block-table entries are the same pool block in all
    of its rows; those blocks are read once per cohort.  The result is the
    same as without cohorts."""
    lib = _lib.load()
    dev = _require_gpu(query, k_pool, v_pool, block_tables, context_lens)
    nb, gn, bs, hd, sb, sh, st = _pool_strides(k_pool, v_pool)
    if query.dim() != 3 or query.shape[2] != hd:
        raise ValueError(f"query must be [b, hn, {hd}], got {tuple(query.shape)}")
    _require_head_dim(hd)
    if query.dtype != k_pool.dtype:
        raise TypeError("query and pools must share a dtype")
    b, hn, _ = query.shape
    if hn % gn != 0:
        raise ValueError(f"{hn} query heads are not a multiple of {gn} KV heads")
    if query.stride(2) != 1 or query.stride(1) != hd:
        query = query.contiguous()
    if block_tables.dtype != torch.int32 or block_tables.dim() != 2 or block_tables.shape[0] != b \
            or block_tables.stride(1) != 1:
        raise ValueError("block_tables must be int32 [b, max_blocks] with contiguous rows")
    if context_lens.dtype != torch.int32 or context_lens.numel() != b or not context_lens.is_contiguous():
        raise ValueError("context_lens must be a contiguous int32 [b] tensor")
    max_context_len = int(max_context_len)
    if max_context_len > block_tables.shape[1] * bs:
        raise ValueError("max_context_len exceeds what the block table can address")
    if out is None:
        out = torch.empty(b, hn * hd, dtype=query.dtype, device=dev)
    elif out.shape != (b, hn * hd) or out.dtype != query.dtype or out.stride(1) != 1:
        raise ValueError("out must be [b, hn*hd] in the query dtype with contiguous rows")
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    cohort_size = int(cohort_size)
    shared_ptr = 0
    if cohort_size > 1:
        n_cohorts = (b + cohort_size - 1) // cohort_size
        if cohort_shared_blocks is None or cohort_shared_blocks.dtype != torch.int32 \
                or cohort_shared_blocks.numel() != n_cohorts or not cohort_shared_blocks.is_contiguous() \
                or cohort_shared_blocks.device != dev:
            raise ValueError(f"cohort_shared_blocks must be a contiguous int32 [{n_cohorts}] tensor on {dev}")
        shared_ptr = cohort_shared_blocks.data_ptr()
    elif cohort_size < 1:
        raise ValueError("cohort_size must be >= 1")
    need = lib.ic_paged_decode_shared_workspace_bytes(b, hn, gn, hd, cohort_size)
    if need == 0 and b > 0:
        raise ValueError(f"cohort_size {cohort_size} with {hn // gn} query heads per KV head is not supported")
    ws = _workspace.get(dev, need)
    if key_mask is not None:
        if key_mask.dtype != torch.uint8 or key_mask.dim() != 3 or key_mask.shape[0] != b \
                or key_mask.shape[1] not in (1, hn) or key_mask.shape[2] < max_context_len \
                or not key_mask.is_contiguous() or key_mask.device != dev:
            raise ValueError(f"key_mask must be a contiguous uint8 [{b}, 1 or {hn}, >= {max_context_len}] tensor")
        if cohort_size != 1:
            raise ValueError("key_mask and cohorts do not combine")
        with torch.cuda.device(dev):
            rc = lib.ic_paged_decode_masked(out.data_ptr(), out.stride(0), query.data_ptr(), query.stride(0),
                                            k_pool.data_ptr(), v_pool.data_ptr(), sb, sh, st,
                                            block_tables.data_ptr(), block_tables.stride(0),
                                            context_lens.data_ptr(), b, hn, gn, hd, bs, nb, max_context_len,
                                            float(scale), min_chunk_tokens, key_mask.data_ptr(),
                                            key_mask.stride(0), key_mask.stride(1) if key_mask.shape[1] > 1 else 0,
                                            ws.data_ptr(), ws.numel(),
                                            _lib.dtype_code(query.dtype), _lib.current_stream_ptr(dev))
        _lib.check("ic_paged_decode_masked", rc)
        return out
    with torch.cuda.device(dev):
        rc = lib.ic_paged_decode_shared(out.data_ptr(), out.stride(0), query.data_ptr(), query.stride(0),
                                        k_pool.data_ptr(), v_pool.data_ptr(), sb, sh, st,
                                        block_tables.data_ptr(), block_tables.stride(0),
                                        context_lens.data_ptr(), b, hn, gn, hd, bs, nb, max_context_len,
                                        float(scale), min_chunk_tokens, cohort_size, shared_ptr,
                                        ws.data_ptr(), ws.numel(),
                                        _lib.dtype_code(query.dtype), _lib.current_stream_ptr(dev))
    _lib.check("ic_paged_decode_shared", rc)
    return out


def paged_decode_static(query: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                        block_tables: torch.Tensor, context_lens: torch.Tensor, max_context_len: int,
                        out: torch.Tensor, scale: float | None = None, min_chunk_tokens: int = 0) -> torch.Tensor:
    """``paged_decode`` without any allocation: the split-K workspace is the
    library's own static device array, ``out`` is the caller's.  For callers
    that may not allocate (graph capture, serving loops).  Batches whose
    workspace exceeds the array raise ``PagedLibraryError`` (IC_ERR_STATIC_LIMIT);
    calls that overlap in time on one GPU race on the array."""
    lib = _lib.load()
    dev = _require_gpu(query, k_pool, v_pool, block_tables, context_lens, out)
    nb, gn, bs, hd, sb, sh, st = _pool_strides(k_pool, v_pool)
    if query.dim() != 3 or query.shape[2] != hd or query.stride(2) != 1 or query.stride(1) != hd:
        raise ValueError(f"query must be [b, hn, {hd}] with contiguous heads")
    _require_head_dim(hd)
    if query.dtype != k_pool.dtype:
        raise TypeError("query and pools must share a dtype")
    b, hn, _ = query.shape
    if hn % gn != 0:
        raise ValueError(f"{hn} query heads are not a multiple of {gn} KV heads")
    if block_tables.dtype != torch.int32 or block_tables.dim() != 2 or block_tables.shape[0] != b \
            or block_tables.stride(1) != 1:
        raise ValueError("block_tables must be int32 [b, max_blocks] with contiguous rows")
    if context_lens.dtype != torch.int32 or context_lens.numel() != b or not context_lens.is_contiguous():
        raise ValueError("context_lens must be a contiguous int32 [b] tensor")
    max_context_len = int(max_context_len)
    if max_context_len > block_tables.shape[1] * bs:
        raise ValueError("max_context_len exceeds what the block table can address")
    if out.shape != (b, hn * hd) or out.dtype != query.dtype or out.stride(1) != 1:
        raise ValueError("out must be [b, hn*hd] in the query dtype with contiguous rows")
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    with torch.cuda.device(dev):
        rc = lib.ic_paged_decode_static(out.data_ptr(), out.stride(0), query.data_ptr(), query.stride(0),
                                        k_pool.data_ptr(), v_pool.data_ptr(), sb, sh, st,
                                        block_tables.data_ptr(), block_tables.stride(0),
                                        context_lens.data_ptr(), b, hn, gn, hd, bs, nb, max_context_len,
                                        float(scale), min_chunk_tokens,
                                        _lib.dtype_code(query.dtype), _lib.current_stream_ptr(dev))
    _lib.check("ic_paged_decode_static", rc)
    return out


def shared_prefix_blocks(block_tables, context_lens, block_size: int, cohort_size: int):
    """Host-side helper: for each cohort of ``cohort_size`` consecutive rows of
    ``block_tables`` (numpy or CPU tensor, ``[b, max_blocks]``), the number of
    leading entries that are equal in all its rows and lie within every row's
    context.  Returns an int32 numpy array ``[ceil(b / cohort_size)]``."""
    import numpy as np
    tables = np.asarray(block_tables)
    ctx = np.asarray(context_lens).astype(np.int64)
    b = tables.shape[0]
    n_cohorts = (b + cohort_size - 1) // cohort_size
    out = np.zeros(n_cohorts, dtype=np.int32)
    for c in range(n_cohorts):
        rows = tables[c * cohort_size:(c + 1) * cohort_size]
        lim = int((ctx[c * cohort_size:(c + 1) * cohort_size] // block_size).min())
        lim = max(min(lim, tables.shape[1]), 0)
        if rows.shape[0] < 2 or lim == 0:
            out[c] = lim if rows.shape[0] == 1 else 0
            continue
        same = (rows[1:, :lim] == rows[:1, :lim]).all(axis=0)
        out[c] = lim if same.all() else int(np.argmin(same))
    return out


def paged_prefill(query: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                  block_tables: torch.Tensor, context_lens: torch.Tensor,
                  cu_seqlens_q: torch.Tensor, max_chunk_len: int, causal: bool = True,
                  scale: float | None = None, out: torch.Tensor | None = None,
                  mask: torch.Tensor | None = None) -> torch.Tensor:
    """Chunked prefill.  ``query`` is the flat ``[n_tokens, hn, hd]``
    concatenation of the sequences' new chunks (chunk ``i`` = rows
    ``cu_seqlens_q[i]:cu_seqlens_q[i+1]``); the chunk's K/V are already in the
    pool and ``context_lens[i]`` counts prefix + chunk.  -> ``[n_tokens, hn*hd]``.

    ``mask`` (uint8 ``[1 or n_seqs, 1 or hn, >= max_chunk_len, keys]``,
    last dimension contiguous) replaces the causal rule: byte (i, h, r, j) == 0
    hides key j from row r of chunk i (head h); a key past the mask's last
    dimension is hidden too (nothing is read beyond it).  Hidden keys get the
    reference's finite fill value: a row that sees nothing averages V."""
    lib = _lib.load()
    dev = _require_gpu(query, k_pool, v_pool, block_tables, context_lens, cu_seqlens_q)
    nb, gn, bs, hd, sb, sh, st = _pool_strides(k_pool, v_pool)
    if query.dim() != 3 or query.shape[2] != hd:
        raise ValueError(f"query must be [n_tokens, hn, {hd}], got {tuple(query.shape)}")
    _require_head_dim(hd)
    if query.dtype != k_pool.dtype:
        raise TypeError("query and pools must share a dtype")
    n_tokens, hn, _ = query.shape
    if hn % gn != 0:
        raise ValueError(f"{hn} query heads are not a multiple of {gn} KV heads")
    if query.stride(2) != 1 or query.stride(1) != hd:
        query = query.contiguous()
    n_seqs = context_lens.numel()
    if block_tables.dtype != torch.int32 or block_tables.dim() != 2 or block_tables.shape[0] != n_seqs \
            or block_tables.stride(1) != 1:
        raise ValueError("block_tables must be int32 [n_seqs, max_blocks] with contiguous rows")
    if context_lens.dtype != torch.int32 or not context_lens.is_contiguous():
        raise ValueError("context_lens must be a contiguous int32 tensor")
    if cu_seqlens_q.dtype != torch.int32 or cu_seqlens_q.numel() != n_seqs + 1 \
            or not cu_seqlens_q.is_contiguous():
        raise ValueError("cu_seqlens_q must be a contiguous int32 [n_seqs + 1] tensor")
    if out is None:
        out = torch.empty(n_tokens, hn * hd, dtype=query.dtype, device=dev)
    elif out.shape != (n_tokens, hn * hd) or out.dtype != query.dtype or out.stride(1) != 1:
        raise ValueError("out must be [n_tokens, hn*hd] in the query dtype with contiguous rows")
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    if mask is not None:
        if mask.dtype != torch.uint8 or mask.dim() != 4 or mask.shape[0] not in (1, n_seqs) \
                or mask.shape[1] not in (1, hn) or mask.shape[2] < max_chunk_len or mask.stride(3) != 1 \
                or mask.device != dev:
            raise ValueError(f"mask must be uint8 [1 or {n_seqs}, 1 or {hn}, >= {max_chunk_len}, keys] on {dev} "
                             "with a contiguous last dimension")
        with torch.cuda.device(dev):
            rc = lib.ic_paged_prefill_masked(out.data_ptr(), out.stride(0), query.data_ptr(), query.stride(0),
                                             k_pool.data_ptr(), v_pool.data_ptr(), sb, sh, st,
                                             block_tables.data_ptr(), block_tables.stride(0),
                                             context_lens.data_ptr(), cu_seqlens_q.data_ptr(), n_seqs,
                                             int(max_chunk_len), hn, gn, hd, bs, nb, float(scale),
                                             mask.data_ptr(),
                                             mask.stride(0) if mask.shape[0] > 1 else 0,
                                             mask.stride(1) if mask.shape[1] > 1 else 0, mask.stride(2),
                                             mask.shape[3], _lib.dtype_code(query.dtype), _lib.current_stream_ptr(dev))
        _lib.check("ic_paged_prefill_masked", rc)
        return out
    with torch.cuda.device(dev):
        rc = lib.ic_paged_prefill(out.data_ptr(), out.stride(0), query.data_ptr(), query.stride(0),
                                  k_pool.data_ptr(), v_pool.data_ptr(), sb, sh, st,
                                  block_tables.data_ptr(), block_tables.stride(0),
                                  context_lens.data_ptr(), cu_seqlens_q.data_ptr(), n_seqs,
                                  int(max_chunk_len), hn, gn, hd, bs, nb, float(scale),
                                  1 if causal else 0, _lib.dtype_code(query.dtype),
                                  _lib.current_stream_ptr(dev))
    _lib.check("ic_paged_prefill", rc)
    return out
