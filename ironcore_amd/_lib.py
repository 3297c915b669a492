"""ctypes binding of libironcore_paged.so (the C ABI in include/ironcore_paged.h).

The library is loaded from ironcore_amd/lib/, built in-tree by
``python -m ironcore_amd.build``.  There is no fallback: if the library is
missing every paged operation raises.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p
from pathlib import Path

import torch

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libironcore_paged.so"

IC_OK = 0
IC_DTYPE = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}

# name -> (restype, argtypes); mirrors include/ironcore_paged.h one to one.
SIGNATURES = {
    "ic_version": (c_int, []),
    "ic_error_string": (c_char_p, [c_int]),
    "ic_mfma_probe": (c_int64, [c_int, c_void_p, c_void_p]),
    "ic_decode_occupancy_queries": (c_int64, []),
    "ic_kv_append": (c_int, [
        c_void_p, c_void_p, c_int64,            # k_new, v_new, new_stride_token
        c_void_p, c_void_p,                     # k_pool, v_pool
        c_int64, c_int64, c_int64,              # pool strides: block, head, token
        c_void_p, c_int64,                      # slot_mapping, n_tokens
        c_int, c_int, c_int, c_int64,           # gn, hd, block_size, num_blocks
        c_int, c_void_p]),                      # dtype, stream
    "ic_rope_kv_append": (c_int, [
        c_void_p, c_int64, c_int,               # q, q_stride_token, hn
        c_void_p, c_void_p, c_int64,            # k_new, v_new, new_stride_token
        c_void_p, c_void_p,                     # k_pool, v_pool
        c_int64, c_int64, c_int64,              # pool strides
        c_void_p, c_void_p,                     # slot_mapping, positions
        c_void_p, c_void_p, c_int64,            # cos_table, sin_table, table_rows
        c_int64, c_int, c_int, c_int,           # n_tokens, gn, hd, block_size
        c_int64, c_int, c_void_p]),             # num_blocks, dtype, stream
    "ic_paged_decode_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "ic_paged_decode": (c_int, [
        c_void_p, c_int64, c_void_p, c_int64,   # out, out_stride, q, q_stride
        c_void_p, c_void_p,                     # k_pool, v_pool
        c_int64, c_int64, c_int64,              # pool strides
        c_void_p, c_int64, c_void_p,            # block_tables, stride, context_lens
        c_int, c_int, c_int, c_int, c_int,      # n_seqs, hn, gn, hd, block_size
        c_int64, c_int, c_float,                # num_blocks, max_context_len, scale
        c_int, c_void_p, c_size_t,              # min_chunk_tokens, workspace, workspace_bytes
        c_int, c_void_p]),                      # dtype, stream
    "ic_paged_decode_shared_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int]),
    "ic_paged_decode_shared": (c_int, [
        c_void_p, c_int64, c_void_p, c_int64,   # out, out_stride, q, q_stride
        c_void_p, c_void_p,                     # k_pool, v_pool
        c_int64, c_int64, c_int64,              # pool strides
        c_void_p, c_int64, c_void_p,            # block_tables, stride, context_lens
        c_int, c_int, c_int, c_int, c_int,      # n_seqs, hn, gn, hd, block_size
        c_int64, c_int, c_float,                # num_blocks, max_context_len, scale
        c_int, c_int, c_void_p,                 # min_chunk_tokens, cohort_size, cohort_shared_blocks
        c_void_p, c_size_t,                     # workspace, workspace_bytes
        c_int, c_void_p]),                      # dtype, stream
    "ic_paged_decode_static_scratch_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "ic_paged_decode_static": (c_int, [
        c_void_p, c_int64, c_void_p, c_int64,   # out, out_stride, q, q_stride
        c_void_p, c_void_p,                     # k_pool, v_pool
        c_int64, c_int64, c_int64,              # pool strides
        c_void_p, c_int64, c_void_p,            # block_tables, stride, context_lens
        c_int, c_int, c_int, c_int, c_int,      # n_seqs, hn, gn, hd, block_size
        c_int64, c_int, c_float,                # num_blocks, max_context_len, scale
        c_int, c_int, c_void_p]),               # min_chunk_tokens, dtype, stream
    "ic_paged_prefill": (c_int, [
        c_void_p, c_int64, c_void_p, c_int64,   # out, out_stride, q, q_stride
        c_void_p, c_void_p,                     # k_pool, v_pool
        c_int64, c_int64, c_int64,              # pool strides
        c_void_p, c_int64, c_void_p, c_void_p,  # block_tables, stride, context_lens, cu_seqlens_q
        c_int, c_int,                           # n_seqs, max_chunk_len
        c_int, c_int, c_int, c_int,             # hn, gn, hd, block_size
        c_int64, c_float, c_int,                # num_blocks, scale, causal
        c_int, c_void_p]),                      # dtype, stream
    "ic_paged_prefill_masked": (c_int, [
        c_void_p, c_int64, c_void_p, c_int64,   # out, out_stride, q, q_stride
        c_void_p, c_void_p,                     # k_pool, v_pool
        c_int64, c_int64, c_int64,              # pool strides
        c_void_p, c_int64, c_void_p, c_void_p,  # block_tables, stride, context_lens, cu_seqlens_q
        c_int, c_int,                           # n_seqs, max_chunk_len
        c_int, c_int, c_int, c_int,             # hn, gn, hd, block_size
        c_int64, c_float,                       # num_blocks, scale
        c_void_p, c_int64, c_int64, c_int64,    # mask, strides: seq, head, row
        c_int64, c_int, c_void_p]),             # mask_keys, dtype, stream
    "ic_paged_decode_masked": (c_int, [
        c_void_p, c_int64, c_void_p, c_int64,   # out, out_stride, q, q_stride
        c_void_p, c_void_p,                     # k_pool, v_pool
        c_int64, c_int64, c_int64,              # pool strides
        c_void_p, c_int64, c_void_p,            # block_tables, stride, context_lens
        c_int, c_int, c_int, c_int, c_int,      # n_seqs, hn, gn, hd, block_size
        c_int64, c_int, c_float,                # num_blocks, max_context_len, scale
        c_int,                                  # min_chunk_tokens
        c_void_p, c_int64, c_int64,             # key_mask, strides: seq, head
        c_void_p, c_size_t,                     # workspace, workspace_bytes
        c_int, c_void_p]),                      # dtype, stream
}


class PagedLibraryError(RuntimeError):
    """A C-ABI call returned a negative IC_ERR_* code."""

    def __init__(self, func: str, code: int, message: str):
        super().__init__(f"{func} failed with code {code}: {message}")
        self.func = func
        self.code = code


_lib = None


def load() -> ctypes.CDLL:
    """Load the shared library (once) and declare every prototype."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m ironcore_amd.build` "
            "(there is no non-HIP fallback for the paged-attention path)")
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(func: str, code: int) -> None:
    if code != IC_OK:
        msg = load().ic_error_string(code).decode()
        raise PagedLibraryError(func, code, msg)


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return IC_DTYPE[dtype]
    except KeyError:
        raise TypeError(f"paged attention supports bf16/fp16/fp32 tensors, got {dtype}") from None


def current_stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream
