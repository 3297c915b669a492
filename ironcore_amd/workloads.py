"""Synthetic paged-attention workloads (the benchmark configurations and
scaled-down versions of them for parity tests).

Everything is seeded.  Integer structure (context lengths, block
permutation) comes from ``numpy.random.default_rng(seed)`` on the host; tensor
contents come from ``torch.Generator`` on the CPU (``device_values=False``,
so a CPU checker and the GPU see the same bits) or on the GPU
(``device_values=True``, for sizes where host generation would dominate).
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch


@dataclass
class DecodeWorkload:
    query: torch.Tensor          # [b, hn, hd]
    k_pool: torch.Tensor         # [num_blocks, gn, B, hd]
    v_pool: torch.Tensor
    block_tables: torch.Tensor   # [b, max_blocks] int32
    context_lens: torch.Tensor   # [b] int32
    max_context_len: int
    hn: int
    gn: int
    hd: int
    block_size: int
    unique_tokens: int           # tokens resident in the pool that the batch reads
    logical_tokens: int          # sum of context lengths
    name: str = ""
    extra: dict = field(default_factory=dict)

    @property
    def batch(self) -> int:
        return self.query.shape[0]

    def kv_bytes_per_token(self) -> int:
        return 2 * self.gn * self.hd * self.query.element_size()

    def algorithmic_bytes(self) -> int:
        """K/V read once per KV head (unique tokens) + Q + O + block-table
        entries + context lengths."""
        es = self.query.element_size()
        n_blk = int(((self.context_lens.cpu().long() + self.block_size - 1) // self.block_size).sum())
        return (self.unique_tokens * self.kv_bytes_per_token()
                + 2 * self.batch * self.hn * self.hd * es + 4 * n_blk + 4 * self.batch)

    def to(self, device) -> "DecodeWorkload":
        kw = dict(self.__dict__)
        for k, v in kw.items():
            if isinstance(v, torch.Tensor):
                kw[k] = v.to(device)
        return DecodeWorkload(**kw)


def _randn(shape, dtype, device, seed, device_values):
    if device_values:
        g = torch.Generator(device=device)
        g.manual_seed(seed)
        return torch.randn(shape, generator=g, device=device, dtype=torch.float32).to(dtype)
    g = torch.Generator()
    g.manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=torch.float32).to(dtype).to(device)


def make_decode_workload(batch: int, hn: int, gn: int, hd: int, ctx_lo: int, ctx_hi: int,
                         block_size: int = 16, dtype=torch.bfloat16, device="cpu", seed: int = 0,
                         device_values: bool = False, extra_blocks: int = 0,
                         name: str = "") -> DecodeWorkload:
    """Independent sequences, context lengths uniform in [ctx_lo, ctx_hi],
    block tables a random permutation of a pool sized to fit all sequences
    (plus ``extra_blocks`` unused ones)."""
    rng = np.random.default_rng(seed)
    ctx = rng.integers(ctx_lo, ctx_hi + 1, size=batch)
    nblk = (ctx + block_size - 1) // block_size
    total = int(nblk.sum()) + extra_blocks
    perm = rng.permutation(total)
    max_blocks = int(nblk.max())
    tables = np.zeros((batch, max_blocks), dtype=np.int32)
    pos = 0
    for i in range(batch):
        tables[i, :nblk[i]] = perm[pos:pos + nblk[i]]
        pos += nblk[i]
    dev = torch.device(device)
    shape = (total, gn, block_size, hd)
    return DecodeWorkload(
        query=_randn((batch, hn, hd), dtype, dev, seed + 1, device_values),
        k_pool=_randn(shape, dtype, dev, seed + 2, device_values),
        v_pool=_randn(shape, dtype, dev, seed + 3, device_values),
        block_tables=torch.from_numpy(tables).to(dev),
        context_lens=torch.from_numpy(ctx.astype(np.int32)).to(dev),
        max_context_len=int(ctx.max()), hn=hn, gn=gn, hd=hd, block_size=block_size,
        unique_tokens=int(ctx.sum()), logical_tokens=int(ctx.sum()), name=name)


def make_grpo_workload(n_prompts: int, n_samples: int, hn: int, gn: int, hd: int,
                       prefix_len: int, suffix_lo: int, suffix_hi: int, block_size: int = 16,
                       dtype=torch.bfloat16, device="cpu", seed: int = 0,
                       device_values: bool = False, name: str = "") -> DecodeWorkload:
    """GRPO rollout decode: each group of ``n_samples`` sequences aliases the
    same block-aligned prompt-prefix blocks and has a private suffix of length
    uniform in [suffix_lo, suffix_hi]."""
    if prefix_len % block_size:
        raise ValueError("the shared prefix must be block aligned")
    rng = np.random.default_rng(seed)
    batch = n_prompts * n_samples
    suffix = rng.integers(suffix_lo, suffix_hi + 1, size=batch)
    pre_blk = prefix_len // block_size
    suf_blk = (suffix + block_size - 1) // block_size
    total = n_prompts * pre_blk + int(suf_blk.sum())
    perm = rng.permutation(total)
    max_blocks = pre_blk + int(suf_blk.max())
    tables = np.zeros((batch, max_blocks), dtype=np.int32)
    pos = 0
    prefix_ids = []
    for _ in range(n_prompts):
        prefix_ids.append(perm[pos:pos + pre_blk])
        pos += pre_blk
    for i in range(batch):
        tables[i, :pre_blk] = prefix_ids[i // n_samples]
        tables[i, pre_blk:pre_blk + suf_blk[i]] = perm[pos:pos + suf_blk[i]]
        pos += suf_blk[i]
    ctx = (prefix_len + suffix).astype(np.int32)
    dev = torch.device(device)
    shape = (total, gn, block_size, hd)
    return DecodeWorkload(
        query=_randn((batch, hn, hd), dtype, dev, seed + 1, device_values),
        k_pool=_randn(shape, dtype, dev, seed + 2, device_values),
        v_pool=_randn(shape, dtype, dev, seed + 3, device_values),
        block_tables=torch.from_numpy(tables).to(dev),
        context_lens=torch.from_numpy(ctx).to(dev),
        max_context_len=int(ctx.max()), hn=hn, gn=gn, hd=hd, block_size=block_size,
        unique_tokens=int(n_prompts * prefix_len + suffix.sum()),
        logical_tokens=int(ctx.sum()), name=name,
        extra={"n_prompts": n_prompts, "n_samples": n_samples, "prefix_len": prefix_len})


# ---- the benchmark configurations -------------------------------------------

def llama7b_decode(device="cuda", seed: int = 0, batch: int = 64, ctx_lo: int = 512,
                   ctx_hi: int = 4096, device_values: bool = True) -> DecodeWorkload:
    """Llama-7B layer shape: 32 q heads, 32 kv heads, head_dim 128, bf16, block 16."""
    return make_decode_workload(batch, 32, 32, 128, ctx_lo, ctx_hi, 16, torch.bfloat16, device, seed,
                                device_values, name="llama7b_decode_bs64_ctx512-4096")


def llama70b_gqa_decode(device="cuda", seed: int = 0, batch: int = 128, ctx_lo: int = 1024,
                        ctx_hi: int = 8192, device_values: bool = True) -> DecodeWorkload:
    """Llama-70B attention shape on one GPU: 64 q heads, 8 kv heads, head_dim 128."""
    return make_decode_workload(batch, 64, 8, 128, ctx_lo, ctx_hi, 16, torch.bfloat16, device, seed,
                                device_values, name="llama70b_gqa_decode_bs128_ctx1024-8192")


def qwen7b_grpo_decode(device="cuda", seed: int = 0, n_prompts: int = 32, n_samples: int = 16,
                       device_values: bool = True) -> DecodeWorkload:
    """Qwen-7B-style attention: 28 q heads, 4 kv heads; 32 prompts x 16 samples
    sharing 1024-token prefixes, private suffix uniform in [1, 1024]."""
    return make_grpo_workload(n_prompts, n_samples, 28, 4, 128, 1024, 1, 1024, 16, torch.bfloat16,
                              device, seed, device_values, name="qwen7b_grpo_decode_32x16")


@dataclass
class PrefillWorkload:
    query: torch.Tensor          # [n_tokens, hn, hd]   new chunks, concatenated
    k_new: torch.Tensor          # [n_tokens, gn, hd]   K rows of the new chunks
    v_new: torch.Tensor
    slot_mapping: torch.Tensor   # [n_tokens] int64
    k_pool: torch.Tensor         # [num_blocks, gn, B, hd]; prefixes resident, chunks not yet
    v_pool: torch.Tensor
    block_tables: torch.Tensor   # [n_seqs, max_blocks] int32
    context_lens: torch.Tensor   # [n_seqs] int32   prefix + chunk
    cu_seqlens_q: torch.Tensor   # [n_seqs + 1] int32
    max_chunk_len: int
    hn: int
    gn: int
    hd: int
    block_size: int
    prefix_lens: list
    chunk_lens: list
    name: str = ""

    def flops(self) -> int:
        """2 flops per MAC, QK^T and PV, visible (query, key) pairs only."""
        pairs = sum(c * p + c * (c + 1) // 2 for p, c in zip(self.prefix_lens, self.chunk_lens))
        return 4 * self.hn * self.hd * pairs

    def to(self, device) -> "PrefillWorkload":
        kw = dict(self.__dict__)
        for k, v in kw.items():
            if isinstance(v, torch.Tensor):
                kw[k] = v.to(device)
        return PrefillWorkload(**kw)


def make_prefill_workload(n_seqs: int, hn: int, gn: int, hd: int, prefix_lo: int, prefix_hi: int,
                          chunk_lo: int, chunk_hi: int, block_size: int = 16, dtype=torch.bfloat16,
                          device="cpu", seed: int = 0, device_values: bool = False,
                          name: str = "") -> PrefillWorkload:
    """Each sequence has a cached prefix uniform in [prefix_lo, prefix_hi] and a
    new query chunk uniform in [chunk_lo, chunk_hi]; blocks are a random
    permutation of a pool sized to fit prefix + chunk of every sequence."""
    rng = np.random.default_rng(seed)
    prefix = rng.integers(prefix_lo, prefix_hi + 1, size=n_seqs)
    chunk = rng.integers(chunk_lo, chunk_hi + 1, size=n_seqs)
    total = prefix + chunk
    nblk = (total + block_size - 1) // block_size
    n_blocks = max(int(nblk.sum()), 1)
    perm = rng.permutation(n_blocks)
    max_blocks = max(int(nblk.max()), 1)
    tables = np.zeros((n_seqs, max_blocks), dtype=np.int32)
    slots = []
    pos = 0
    for i in range(n_seqs):
        tables[i, :nblk[i]] = perm[pos:pos + nblk[i]]
        pos += nblk[i]
        for t in range(prefix[i], total[i]):
            slots.append(int(tables[i, t // block_size]) * block_size + t % block_size)
    n_tokens = int(chunk.sum())
    cu = np.concatenate([[0], np.cumsum(chunk)]).astype(np.int32)
    dev = torch.device(device)
    shape = (n_blocks, gn, block_size, hd)
    return PrefillWorkload(
        query=_randn((n_tokens, hn, hd), dtype, dev, seed + 1, device_values),
        k_new=_randn((n_tokens, gn, hd), dtype, dev, seed + 4, device_values),
        v_new=_randn((n_tokens, gn, hd), dtype, dev, seed + 5, device_values),
        slot_mapping=torch.tensor(slots, dtype=torch.int64).to(dev),
        k_pool=_randn(shape, dtype, dev, seed + 2, device_values),
        v_pool=_randn(shape, dtype, dev, seed + 3, device_values),
        block_tables=torch.from_numpy(tables).to(dev),
        context_lens=torch.from_numpy(total.astype(np.int32)).to(dev),
        cu_seqlens_q=torch.from_numpy(cu).to(dev),
        max_chunk_len=int(chunk.max()) if n_seqs else 0, hn=hn, gn=gn, hd=hd, block_size=block_size,
        prefix_lens=[int(x) for x in prefix], chunk_lens=[int(x) for x in chunk], name=name)


def llama7b_chunked_prefill(device="cuda", seed: int = 0, n_seqs: int = 16, chunk: int = 512,
                            prefix_hi: int = 4096, device_values: bool = True) -> PrefillWorkload:
    """Llama-7B dims: 32 heads, head_dim 128, bf16; 16 sequences, cached prefix
    uniform in [0, 4096], new 512-token chunk each, block 16."""
    return make_prefill_workload(n_seqs, 32, 32, 128, 0, prefix_hi, chunk, chunk, 16, torch.bfloat16,
                                 device, seed, device_values, name="llama7b_chunked_prefill_16x512")
