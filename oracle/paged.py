"""Paged drivers for the dense oracle (TEST INFRASTRUCTURE, not product code).

The reference has no KV cache; the block-KV-cache interface below is the one
this build defines, and the oracle's job is to say what any correct
implementation of it must return: the reference's dense attention
(ironcore/layers/attention.py:68-142) applied to the rows the block table
points at.

Cache interface
---------------
k_pool, v_pool   [num_blocks, gn, B, hd]   one block holds B consecutive tokens
                                            of one sequence, all KV heads
block_tables     [b, max_blocks] int32      entry j of row i is the pool block
                                            holding tokens [j*B, (j+1)*B) of
                                            sequence i; rows may alias blocks
context_lens     [b] int32                  tokens visible to the query
                                            (including any just appended)
slot_mapping     [n] int64                  block*B + offset for each new row

Token p of sequence i lives at pool[block_tables[i, p // B], :, p % B, :].
"""
from __future__ import annotations

import torch

from .dense_attention import causal_offset_mask, dense_attention


def kv_append(k_pool: torch.Tensor, v_pool: torch.Tensor, k_new: torch.Tensor,
              v_new: torch.Tensor, slot_mapping: torch.Tensor) -> None:
    """Closed form of the append: row t of k_new/v_new ([n, gn, hd], the K/V a
    transformer layer produced for token t, ironcore/models/transformer.py:
    88-98) is copied bit for bit to its slot.  In place.  Negative slots are
    skipped (padding tokens)."""
    nb, gn, B, hd = k_pool.shape
    for t in range(slot_mapping.numel()):
        s = int(slot_mapping[t])
        if s < 0:
            continue
        blk, off = divmod(s, B)
        k_pool[blk, :, off, :] = k_new[t]
        v_pool[blk, :, off, :] = v_new[t]


def gather_kv(pool: torch.Tensor, block_table_row: torch.Tensor, ctx: int) -> torch.Tensor:
    """Rows 0..ctx-1 of one sequence as a dense [1, ctx, gn, hd] tensor."""
    nb, gn, B, hd = pool.shape
    n_blk = (ctx + B - 1) // B
    blocks = pool[block_table_row[:n_blk].long()]          # [n_blk, gn, B, hd]
    rows = blocks.permute(0, 2, 1, 3).reshape(n_blk * B, gn, hd)
    return rows[:ctx].unsqueeze(0)


def paged_decode(query: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                 block_tables: torch.Tensor, context_lens: torch.Tensor) -> torch.Tensor:
    """One query token per sequence.  query [b, hn, hd] -> [b, hn*hd].
    Per sequence: gather, then the dense oracle with sq = 1 and no mask (a
    single query at the last position sees every cached key)."""
    outs = []
    for i in range(query.shape[0]):
        ctx = int(context_lens[i])
        k = gather_kv(k_pool, block_tables[i], ctx)
        v = gather_kv(v_pool, block_tables[i], ctx)
        outs.append(dense_attention(query[i][None, None], k, v, None)[0, 0])
    return torch.stack(outs)


def paged_prefill(query: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                  block_tables: torch.Tensor, context_lens: torch.Tensor,
                  cu_seqlens_q: torch.Tensor) -> torch.Tensor:
    """Chunked prefill.  query is the flat [n_tokens, hn, hd] concatenation of
    each sequence's new chunk (rows cu_seqlens_q[i]..cu_seqlens_q[i+1]); the
    chunk's K/V are already in the pool and context_lens[i] = prefix + chunk.
    Query row r of a chunk of length C sees keys j <= (ctx - C) + r, the
    causal mask of ironcore/language_model.py:109-114 shifted by the cached
    prefix.  Returns [n_tokens, hn*hd]."""
    outs = []
    for i in range(context_lens.numel()):
        lo, hi = int(cu_seqlens_q[i]), int(cu_seqlens_q[i + 1])
        if hi == lo:
            continue
        ctx = int(context_lens[i])
        k = gather_kv(k_pool, block_tables[i], ctx)
        v = gather_kv(v_pool, block_tables[i], ctx)
        mask = causal_offset_mask(hi - lo, ctx)
        outs.append(dense_attention(query[lo:hi][None], k, v, mask)[0])
    return torch.cat(outs, dim=0)
