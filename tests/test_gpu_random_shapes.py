"""Seeded random shapes through the C ABI against the CPU oracle.

The other GPU files pick their shapes by hand (boundaries, the benchmark
shapes); here a fixed seed draws head counts, head dims, element types, block
sizes, batch sizes and length ranges, so that combinations nobody thought of
are held to the same bars: append bit-exact, attention within 2e-2 (16-bit) or
2e-5 (fp32) of the oracle, the cohort entry point within one bf16 step of the
plain one (how short contexts bend the first bar: parity_bars.py).
Every case prints its parameters before it runs."""
import numpy as np
import pytest
import torch

from ironcore_amd import paged_ops, workloads
from oracle import paged as oracle_paged
from parity_bars import hold as _hold

pytestmark = pytest.mark.gpu

HEADS = [(1, 1), (2, 1), (3, 1), (4, 4), (6, 2), (8, 8), (8, 1), (9, 3), (12, 4), (14, 2), (16, 1), (16, 16),
         (20, 4), (28, 4), (32, 8), (40, 8), (48, 3)]
DTYPES = [torch.bfloat16, torch.bfloat16, torch.float16, torch.float32]


def _f64(*tensors):
    return [t.double() for t in tensors]


def _draw_decode(rng, dims=(64, 128)):
    hn, gn = HEADS[rng.integers(len(HEADS))]
    hd = int(rng.choice(dims))
    dtype = DTYPES[rng.integers(len(DTYPES))]
    block = int(rng.choice([16, 16, 32, 64]))
    batch = int(rng.choice([1, 2, 3, 7, 16, 33, 90]))
    hi = int(rng.choice([1, 20, 130, 600, 2100]))
    lo = int(rng.integers(1, hi + 1))
    return hn, gn, hd, dtype, block, batch, lo, hi


@pytest.mark.parametrize("case", range(80))
def test_random_decode(gpu, case):
    _random_decode(gpu, case, np.random.default_rng(1000 + case))


@pytest.mark.parametrize("case", range(24))
def test_random_decode_head_dim_32(gpu, case):
    _random_decode(gpu, 4000 + case, np.random.default_rng(4000 + case), dims=(32,))


def _random_decode(gpu, case, rng, dims=(64, 128)):
    hn, gn, hd, dtype, block, batch, lo, hi = _draw_decode(rng, dims)
    min_chunk = int(rng.choice([16, 64, 512, 1 << 20]))
    print(f"decode case {case}: hn {hn} gn {gn} hd {hd} {dtype} block {block} batch {batch} ctx [{lo}, {hi}] "
          f"min_chunk_tokens {min_chunk}", flush=True)
    wl = workloads.make_decode_workload(batch, hn, gn, hd, lo, hi, block_size=block, dtype=dtype, seed=case,
                                        extra_blocks=int(rng.integers(0, 4)))
    d = wl.to(gpu)
    out = paged_ops.paged_decode(d.query, d.k_pool, d.v_pool, d.block_tables, d.context_lens, d.max_context_len,
                                 min_chunk_tokens=min_chunk)
    torch.cuda.synchronize()
    ref = oracle_paged.paged_decode(wl.query, wl.k_pool, wl.v_pool, wl.block_tables, wl.context_lens)
    truth = oracle_paged.paged_decode(*_f64(wl.query, wl.k_pool, wl.v_pool), wl.block_tables, wl.context_lens)
    _hold(out, ref, truth, dtype, int(wl.context_lens.min()), f"decode case {case}")


@pytest.mark.parametrize("case", range(48))
def test_random_cohorts(gpu, case):
    _random_cohorts(gpu, case, np.random.default_rng(2000 + case))


@pytest.mark.parametrize("case", range(16))
def test_random_cohorts_head_dim_32(gpu, case):
    _random_cohorts(gpu, 5000 + case, np.random.default_rng(5000 + case), dims=(32,))


def _random_cohorts(gpu, case, rng, dims=(64, 128)):
    hn, gn = HEADS[rng.integers(len(HEADS))]
    hd = int(rng.choice(dims))
    dtype = [torch.bfloat16, torch.float16][rng.integers(2)]
    block = int(rng.choice([16, 16, 32, 64]))
    group = hn // gn
    per_wave = 16 // group
    # cohort sizes the entry point takes: up to 8 waves of 16 / group members each
    cohort = int(rng.integers(2, 8 * per_wave + 1))
    n_samples = int(rng.choice([cohort, cohort, 2 * cohort, max(2, cohort - 1), 5]))
    n_prompts = int(rng.integers(1, 5))
    prefix = block * int(rng.integers(1, 12))
    hi = int(rng.choice([1, 40, 300]))
    print(f"cohort case {case}: hn {hn} gn {gn} hd {hd} {dtype} block {block} prompts {n_prompts} x {n_samples} "
          f"prefix {prefix} suffix [1, {hi}] cohort {cohort}", flush=True)
    wl = workloads.make_grpo_workload(n_prompts, n_samples, hn, gn, hd, prefix, 1, hi, block_size=block, dtype=dtype,
                                      seed=case)
    d = wl.to(gpu)
    shared = paged_ops.shared_prefix_blocks(wl.block_tables.numpy(), wl.context_lens.numpy(), block, cohort)
    plain = paged_ops.paged_decode(d.query, d.k_pool, d.v_pool, d.block_tables, d.context_lens, d.max_context_len)
    out = paged_ops.paged_decode(d.query, d.k_pool, d.v_pool, d.block_tables, d.context_lens, d.max_context_len,
                                 cohort_size=cohort,
                                 cohort_shared_blocks=torch.from_numpy(np.ascontiguousarray(shared, np.int32)).to(gpu))
    torch.cuda.synchronize()
    ref = oracle_paged.paged_decode(wl.query, wl.k_pool, wl.v_pool, wl.block_tables, wl.context_lens)
    truth = oracle_paged.paged_decode(*_f64(wl.query, wl.k_pool, wl.v_pool), wl.block_tables, wl.context_lens)
    _hold(out, ref, truth, dtype, int(wl.context_lens.min()), f"cohort case {case}")
    # the two entry points split and merge in different orders: one step of bf16 at the value's magnitude
    step = torch.maximum(torch.full_like(plain.float(), 4e-3), plain.float().abs() / 128)
    same = ((out.float() - plain.float()).abs() - step).max().item()
    assert same <= 0, f"vs plain decode: {same} beyond one bf16 step"


@pytest.mark.parametrize("case", range(48))
def test_random_prefill(gpu, case):
    _random_prefill(gpu, case, np.random.default_rng(3000 + case))


@pytest.mark.parametrize("case", range(16))
def test_random_prefill_head_dim_32(gpu, case):
    _random_prefill(gpu, 6000 + case, np.random.default_rng(6000 + case), dims=(32,))


@pytest.mark.parametrize("case", range(24))
def test_random_prefill_block_sizes_beyond_powers_of_two(gpu, case):
    """16-bit pools whose blocks are multiples of 16 that are no power of two (the block of a row
    by the reciprocal multiplication, groups that start inside a block), all three head dims."""
    _random_prefill(gpu, 8000 + case, np.random.default_rng(8000 + case), dims=(32, 64, 128),
                    blocks=(48, 80, 96, 112, 144, 176))


@pytest.mark.parametrize("case", range(32))
def test_random_prefill_fp32(gpu, case):
    """fp32 pools (the fp32 matrix-instruction kernel), all three head dims, block sizes that are no
    power of two among them."""
    _random_prefill(gpu, 7000 + case, np.random.default_rng(7000 + case), dims=(32, 64, 128),
                    dtypes=(torch.float32,), blocks=(16, 16, 32, 48, 64, 80))


def _random_prefill(gpu, case, rng, dims=(64, 128), dtypes=(torch.bfloat16, torch.bfloat16, torch.float16),
                    blocks=(16, 16, 32, 64)):
    hn, gn = HEADS[rng.integers(len(HEADS))]
    hd = int(rng.choice(dims))
    dtype = dtypes[rng.integers(len(dtypes))]
    block = int(rng.choice(blocks))
    n_seqs = int(rng.choice([1, 2, 5, 9]))
    p_hi = int(rng.choice([0, 30, 300, 900]))
    c_hi = int(rng.choice([1, 40, 260, 520]))
    c_lo = int(rng.integers(0, c_hi + 1))
    if hn * n_seqs * (p_hi + c_hi) * c_hi > 6e7:       # keep the CPU oracle within seconds
        n_seqs = 2
    print(f"prefill case {case}: hn {hn} gn {gn} hd {hd} {dtype} block {block} seqs {n_seqs} prefix [0, {p_hi}] "
          f"chunk [{c_lo}, {c_hi}]", flush=True)
    seed = case
    while True:   # a draw of empty chunks only tests nothing: take the next seed that has a query row
        wl = workloads.make_prefill_workload(n_seqs, hn, gn, hd, 0, p_hi, c_lo, c_hi, block_size=block, dtype=dtype,
                                             seed=seed)
        if wl.query.shape[0] > 0:
            break
        seed += 1000
    d = wl.to(gpu)
    paged_ops.kv_append(d.k_new, d.v_new, d.k_pool, d.v_pool, d.slot_mapping)
    out = paged_ops.paged_prefill(d.query, d.k_pool, d.v_pool, d.block_tables, d.context_lens, d.cu_seqlens_q,
                                  d.max_chunk_len)
    torch.cuda.synchronize()
    kp, vp = wl.k_pool.clone(), wl.v_pool.clone()
    oracle_paged.kv_append(kp, vp, wl.k_new, wl.v_new, wl.slot_mapping)
    bits = torch.int32 if dtype == torch.float32 else torch.int16
    assert torch.equal(d.k_pool.cpu().view(bits), kp.view(bits)), "append not bit-exact"
    assert torch.equal(d.v_pool.cpu().view(bits), vp.view(bits)), "append not bit-exact"
    ref = oracle_paged.paged_prefill(wl.query, kp, vp, wl.block_tables, wl.context_lens, wl.cu_seqlens_q)
    truth = oracle_paged.paged_prefill(*_f64(wl.query, kp, vp), wl.block_tables, wl.context_lens, wl.cu_seqlens_q)
    # the first row of a chunk sees its prefix and itself
    min_ctx = min(p + 1 for p, c in zip(wl.prefix_lens, wl.chunk_lens) if c > 0)
    _hold(out, ref, truth, dtype, min_ctx, f"prefill case {case}")
