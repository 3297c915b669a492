"""Block KV cache: pools, block allocator with prefix sharing, batch metadata.

The reference has no KV cache (its only generation loop recomputes the whole
sequence every step, examples/generate_text.py:24-40), so this interface is
defined here.  One ``PagedKVCache`` serves all layers of a model:

* per layer a K pool and a V pool ``[num_blocks, gn, block_size, hd]``
  (native layout of the kernels: one (block, KV head) tile is contiguous);
* one block table per sequence, shared by all layers (layer ``l`` of a
  sequence uses the same block ids in layer ``l``'s pools);
* a host-side allocator with reference counts, so sequences forked from a
  common prompt (GRPO groups) alias the prompt's full blocks and copy only the
  partly filled last block.

Everything the kernels need per step comes from :meth:`PagedKVCache.prepare`,
which advances the sequences by the step's new tokens and returns a
``PagedAttentionMetadata`` (block tables, context lengths, slot mapping).  The
allocator state lives on the host; ``prepare`` uploads small int tensors and
never reads anything back from the GPU.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Iterable, Sequence

import torch

from .layers.attention import PagedAttentionMetadata


class OutOfBlocks(RuntimeError):
    """The pool has no free block left."""


class BlockAllocator:
    """Free list + reference counts over ``num_blocks`` pool blocks."""

    def __init__(self, num_blocks: int):
        self.num_blocks = num_blocks
        self._free = list(range(num_blocks - 1, -1, -1))
        self._refs = [0] * num_blocks

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self) -> int:
        if not self._free:
            raise OutOfBlocks(f"all {self.num_blocks} KV blocks are in use")
        blk = self._free.pop()
        self._refs[blk] = 1
        return blk

    def share(self, blk: int) -> int:
        if self._refs[blk] <= 0:
            raise ValueError(f"block {blk} is not allocated")
        self._refs[blk] += 1
        return blk

    def release(self, blk: int) -> None:
        if self._refs[blk] <= 0:
            raise ValueError(f"block {blk} is not allocated")
        self._refs[blk] -= 1
        if self._refs[blk] == 0:
            self._free.append(blk)

    def ref_count(self, blk: int) -> int:
        return self._refs[blk]


@dataclass
class _Sequence:
    blocks: list = field(default_factory=list)
    length: int = 0


class PagedKVCache:
    """Pools for ``num_layers`` layers plus the sequences that live in them."""

    def __init__(self, num_layers: int, num_blocks: int, block_size: int, num_kv_heads: int,
                 head_dim: int, dtype: torch.dtype, device):
        if block_size % 16 != 0:
            raise ValueError("block_size must be a multiple of 16 (the kernels walk 16-token tiles)")
        self.num_layers = num_layers
        self.num_blocks = num_blocks
        self.block_size = block_size
        self.device = torch.device(device)
        shape = (num_layers, num_blocks, num_kv_heads, block_size, head_dim)
        self.k_pools = torch.zeros(shape, dtype=dtype, device=self.device)
        self.v_pools = torch.zeros(shape, dtype=dtype, device=self.device)
        self.allocator = BlockAllocator(num_blocks)
        self._seqs: dict[int, _Sequence] = {}
        self._next_id = 0

    # ---- pools -----------------------------------------------------------------
    def layer(self, index: int):
        """(k_pool, v_pool) of one layer, the ``kv_cache`` argument of
        ``Attention.forward``."""
        return self.k_pools[index], self.v_pools[index]

    # ---- sequences ---------------------------------------------------------------
    def add_sequence(self) -> int:
        sid = self._next_id
        self._next_id += 1
        self._seqs[sid] = _Sequence()
        return sid

    def length(self, sid: int) -> int:
        return self._seqs[sid].length

    def blocks(self, sid: int) -> list:
        return list(self._seqs[sid].blocks)

    def free_sequence(self, sid: int) -> None:
        for blk in self._seqs.pop(sid).blocks:
            self.allocator.release(blk)

    def fork(self, sid: int) -> int:
        """New sequence with the same content: full blocks are aliased
        (reference count up), a partly filled last block is copied so that the
        two sequences can append independently."""
        src = self._seqs[sid]
        if src.length % self.block_size and self.allocator.num_free < 1:
            raise OutOfBlocks("no free KV block for the copy of the partly filled block")
        child = _Sequence(length=src.length)
        full = src.length // self.block_size
        for blk in src.blocks[:full]:
            child.blocks.append(self.allocator.share(blk))
        if src.length % self.block_size:
            new = self.allocator.allocate()
            old = src.blocks[full]
            self.k_pools[:, new].copy_(self.k_pools[:, old])
            self.v_pools[:, new].copy_(self.v_pools[:, old])
            child.blocks.append(new)
        cid = self._next_id
        self._next_id += 1
        self._seqs[cid] = child
        return cid

    def _blocks_needed(self, seq: _Sequence, new_tokens: int) -> int:
        """Blocks the allocator must still give for ``new_tokens`` more tokens:
        new ones past the blocks the sequence holds, plus the private copy of a
        shared block that the next token would be written into."""
        if new_tokens <= 0:
            return 0
        bs = self.block_size
        need = max((seq.length + new_tokens + bs - 1) // bs - len(seq.blocks), 0)
        idx = seq.length // bs
        if idx < len(seq.blocks) and self.allocator.ref_count(seq.blocks[idx]) > 1:
            need += 1
        return need

    def _slot_for_append(self, seq: _Sequence) -> int:
        """Slot of the next token; allocates a block at block boundaries and
        un-shares an aliased block before it is written (copy on write)."""
        bs = self.block_size
        idx, off = divmod(seq.length, bs)
        if idx == len(seq.blocks):
            seq.blocks.append(self.allocator.allocate())
        blk = seq.blocks[idx]
        if self.allocator.ref_count(blk) > 1:
            new = self.allocator.allocate()
            self.k_pools[:, new].copy_(self.k_pools[:, blk])
            self.v_pools[:, new].copy_(self.v_pools[:, blk])
            self.allocator.release(blk)
            seq.blocks[idx] = blk = new
        seq.length += 1
        return blk * bs + off

    # ---- decoding without per-step host work ---------------------------------------------
    def reserve(self, sid: int, total_length: int) -> None:
        """Give the sequence every block it needs to grow to ``total_length``
        tokens, and un-share the block its next token goes to, so that the
        following appends need nothing from the host (a captured graph can
        compute their slots on the device from :meth:`block_table`)."""
        seq = self._seqs[sid]
        bs = self.block_size
        need = self._blocks_needed(seq, max(total_length - seq.length, 0))
        if need > self.allocator.num_free:
            raise OutOfBlocks(f"{need} KV blocks needed, {self.allocator.num_free} free")
        idx, off = divmod(seq.length, bs)
        if off and self.allocator.ref_count(seq.blocks[idx]) > 1:
            new = self.allocator.allocate()
            old = seq.blocks[idx]
            self.k_pools[:, new].copy_(self.k_pools[:, old])
            self.v_pools[:, new].copy_(self.v_pools[:, old])
            self.allocator.release(old)
            seq.blocks[idx] = new
        while len(seq.blocks) * bs < total_length:
            seq.blocks.append(self.allocator.allocate())

    def block_table(self, seq_ids: Sequence[int]) -> torch.Tensor:
        """int32 ``[n, max_blocks]`` device table of all blocks the sequences
        hold, reserved ones included (rows padded with block 0)."""
        width = max((len(self._seqs[s].blocks) for s in seq_ids), default=1) or 1
        table = [self._seqs[s].blocks + [0] * (width - len(self._seqs[s].blocks)) for s in seq_ids]
        return torch.tensor(table, dtype=torch.int32, device=self.device).view(len(seq_ids), width)

    def advance(self, seq_ids: Sequence[int], n_tokens: int) -> None:
        """Record that ``n_tokens`` rows per sequence were appended into
        reserved blocks by device-side bookkeeping."""
        for sid in seq_ids:
            seq = self._seqs[sid]
            if seq.length + n_tokens > len(seq.blocks) * self.block_size:
                raise ValueError("tokens were appended beyond the reserved blocks")
            seq.length += n_tokens

    # ---- per-step metadata -----------------------------------------------------------
    def prepare(self, seq_ids: Sequence[int], new_tokens: int | Iterable[int],
                cohort_size: int = 1) -> PagedAttentionMetadata:
        """Advance each sequence by its number of new tokens (one int for all,
        or one per sequence: the step's tensors are then ``[b, longest, ...]``
        with the rows a sequence does not have as padding, slot -1) and build
        the step's metadata.  The new K/V rows must then be passed through
        ``Attention.forward(..., kv_cache=cache.layer(l), attn_metadata=meta)``
        for every layer; the same metadata serves all layers.

        ``cohort_size`` > 1 groups consecutive ``seq_ids`` into cohorts and
        records how many leading blocks each cohort's members alias (forks of
        one prompt listed next to each other), so decode streams them once."""
        n = len(seq_ids)
        counts = [new_tokens] * n if isinstance(new_tokens, int) else list(new_tokens)
        if len(counts) != n:
            raise ValueError("one new-token count per sequence")
        width = max(counts) if counts else 0
        ragged = any(c != width for c in counts)
        if ragged and cohort_size > 1:
            raise ValueError("cohorts are a decode feature: one new token per sequence")
        # all or nothing: a step that does not fit leaves every sequence as it was
        need = sum(self._blocks_needed(self._seqs[sid], c) for sid, c in zip(seq_ids, counts))
        if need > self.allocator.num_free:
            raise OutOfBlocks(f"{need} KV blocks needed for this step, {self.allocator.num_free} free")
        slots, positions = [], []
        for sid, c in zip(seq_ids, counts):
            seq = self._seqs[sid]
            start = seq.length
            row = [self._slot_for_append(seq) for _ in range(c)]
            slots.extend(row + [-1] * (width - c))
            positions.extend(list(range(start, start + c)) + [0] * (width - c))
        lens = [self._seqs[s].length for s in seq_ids]
        max_blocks = max((len(self._seqs[s].blocks) for s in seq_ids), default=1) or 1
        table = [self._seqs[s].blocks + [0] * (max_blocks - len(self._seqs[s].blocks)) for s in seq_ids]
        dev = self.device
        cu = chunk_rows = None
        if ragged:
            # rows are padded to `width` ([b, width, ...] tensors); the kernels get the true bounds
            # and the layer packs the rows that exist
            bounds = [0]
            for c in counts:
                bounds.append(bounds[-1] + c)
            cu = torch.tensor(bounds, dtype=torch.int32, device=dev)
            chunk_rows = torch.tensor([i * width + t for i, c in enumerate(counts) for t in range(c)],
                                      dtype=torch.int64, device=dev)
        shared = None
        if cohort_size > 1 and n > 0:
            from .paged_ops import shared_prefix_blocks
            shared = torch.from_numpy(shared_prefix_blocks(table, lens, self.block_size, cohort_size)).to(dev)
        return PagedAttentionMetadata(
            block_tables=torch.tensor(table, dtype=torch.int32, device=dev).view(n, max_blocks),
            context_lens=torch.tensor(lens, dtype=torch.int32, device=dev),
            slot_mapping=torch.tensor(slots, dtype=torch.int64, device=dev),
            max_context_len=max(lens, default=0),
            cu_seqlens_q=cu,
            cohort_size=cohort_size if shared is not None else 1,
            cohort_shared_blocks=shared,
            positions=torch.tensor(positions, dtype=torch.int32, device=dev),
            chunk_rows=chunk_rows, max_chunk_len=width)
