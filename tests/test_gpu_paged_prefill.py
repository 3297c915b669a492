"""Chunked prefill (the 16-bit and the fp32 matrix-core kernels) through the C
ABI against the CPU oracle: the reference's dense attention with the offset
causal mask on the gathered rows.  Tolerance: max-abs 2e-2 (bf16/fp16), the
bound the target states; 1e-4 for fp32 pools."""
import pytest
import torch

from ironcore_amd import paged_ops, workloads
from oracle import paged as oracle_paged

pytestmark = pytest.mark.gpu
TOL = 2e-2
FP32_TOL = 1e-4


def _run(wl, gpu, causal=True):
    d = wl.to(gpu)
    paged_ops.kv_append(d.k_new, d.v_new, d.k_pool, d.v_pool, d.slot_mapping)
    out = paged_ops.paged_prefill(d.query, d.k_pool, d.v_pool, d.block_tables, d.context_lens,
                                  d.cu_seqlens_q, d.max_chunk_len, causal=causal)
    torch.cuda.synchronize()
    return out.cpu(), d


def _oracle(wl):
    kp, vp = wl.k_pool.clone(), wl.v_pool.clone()
    oracle_paged.kv_append(kp, vp, wl.k_new, wl.v_new, wl.slot_mapping)
    return oracle_paged.paged_prefill(wl.query, kp, vp, wl.block_tables, wl.context_lens, wl.cu_seqlens_q), kp, vp


def _check(wl, gpu, tol=None):
    out, d = _run(wl, gpu)
    ref, kp, vp = _oracle(wl)
    fp32 = wl.query.dtype == torch.float32
    bits = torch.int32 if fp32 else torch.int16
    assert torch.equal(d.k_pool.cpu().view(bits), kp.view(bits)), "append not bit-exact"
    assert torch.equal(d.v_pool.cpu().view(bits), vp.view(bits)), "append not bit-exact"
    assert torch.isfinite(out.float()).all()
    diff = (out.float() - ref.float()).abs().max().item()
    tol = tol or (FP32_TOL if fp32 else TOL)
    assert diff <= tol, f"max|diff| {diff}"
    return diff


@pytest.mark.parametrize("prefix,chunk", [(0, 1), (0, 17), (0, 128), (5, 64), (100, 33), (64, 129),
                                          (300, 200), (1000, 256), (63, 65)])
def test_prefill_prefix_chunk_shapes(gpu, prefix, chunk):
    wl = workloads.make_prefill_workload(2, 4, 4, 128, prefix, prefix, chunk, chunk, seed=prefix + chunk)
    _check(wl, gpu)


@pytest.mark.parametrize("hn,gn", [(8, 8), (8, 2), (8, 1), (28, 4)])
@pytest.mark.parametrize("hd", [32, 64, 128])
def test_prefill_gqa_and_head_dims(gpu, hn, gn, hd):
    wl = workloads.make_prefill_workload(3, hn, gn, hd, 0, 200, 1, 150, seed=hn + gn + hd)
    _check(wl, gpu)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("prefix,chunk,block", [(0, 300, 16), (700, 130, 16), (45, 257, 64)])
def test_prefill_head_dim_32(gpu, dtype, prefix, chunk, block):
    """Head dimension 32: several K/V tiles, two query tiles, both block sizes."""
    wl = workloads.make_prefill_workload(3, 6, 2, 32, prefix, prefix + 40, 1, chunk, block_size=block, dtype=dtype,
                                         seed=prefix + chunk)
    _check(wl, gpu)


@pytest.mark.parametrize("n_seqs", [64, 65, 130])
def test_prefill_many_sequences(gpu, n_seqs):
    """Batches at and beyond one sequence per lane: up to 64 sequences the
    kernel ranks them by context length inside a wave (64 exactly fills it),
    beyond that a workgroup looks its sequence up directly.  Short ragged
    chunks (some empty) behind short prefixes, with equal context lengths among
    them so that the ranking's tie rule decides."""
    wl = workloads.make_prefill_workload(n_seqs, 4, 2, 64, 0, 100, 0, 40, seed=n_seqs)
    lens = wl.context_lens.tolist()
    assert len(set(lens)) < len(lens), "the draw should contain equal context lengths"
    assert 0 in wl.chunk_lens
    _check(wl, gpu)


@pytest.mark.parametrize("block", [48, 80, 112])
def test_prefill_block_sizes_that_are_no_power_of_two(gpu, block):
    """Any multiple of 16 tokens is a block size (the decode kernel and the
    cache take them too): prefill, then a decode step over the same pools."""
    wl = workloads.make_prefill_workload(3, 8, 2, 128, 0, 500, 1, 300, block_size=block, seed=block)
    _check(wl, gpu)
    d = wl.to(gpu)
    paged_ops.kv_append(d.k_new, d.v_new, d.k_pool, d.v_pool, d.slot_mapping)
    last = (d.cu_seqlens_q[1:] - 1).long()
    keep = [i for i, c in enumerate(wl.chunk_lens) if c > 0]
    q = d.query.index_select(0, last[keep])
    dec = paged_ops.paged_decode(q, d.k_pool, d.v_pool, d.block_tables[keep], d.context_lens[keep].contiguous(),
                                 int(wl.context_lens.max()))
    pre = paged_ops.paged_prefill(d.query, d.k_pool, d.v_pool, d.block_tables, d.context_lens, d.cu_seqlens_q,
                                  d.max_chunk_len)
    torch.cuda.synchronize()
    assert (dec.float() - pre.index_select(0, last[keep]).float()).abs().max().item() <= 4e-3


@pytest.mark.parametrize("prefix,chunk", [(0, 1), (0, 17), (0, 128), (5, 64), (100, 33), (64, 129), (300, 200),
                                          (1000, 256), (63, 65), (31, 300)])
def test_prefill_fp32_prefix_chunk_shapes(gpu, prefix, chunk):
    """fp32 pools: 32-token K/V tiles, 128-row query tiles, every product and sum in fp32."""
    wl = workloads.make_prefill_workload(2, 4, 4, 128, prefix, prefix, chunk, chunk, dtype=torch.float32,
                                         seed=prefix + chunk)
    _check(wl, gpu)


@pytest.mark.parametrize("hn,gn", [(8, 8), (8, 2), (6, 1), (28, 4)])
@pytest.mark.parametrize("hd", [32, 64, 128])
def test_prefill_fp32_gqa_and_head_dims(gpu, hn, gn, hd):
    wl = workloads.make_prefill_workload(3, hn, gn, hd, 0, 200, 1, 150, dtype=torch.float32, seed=hn + gn + hd)
    _check(wl, gpu)


@pytest.mark.parametrize("block", [16, 48, 64, 80])
def test_prefill_fp32_block_sizes_ragged_batch(gpu, block):
    """Ragged chunks (one of them empty) over several block sizes, among them ones that are no
    power of two."""
    wl = workloads.make_prefill_workload(6, 4, 2, 64, 0, 300, 0, 200, block_size=block, dtype=torch.float32,
                                         seed=block)
    _check(wl, gpu)


def test_prefill_fp32_many_sequences_and_garbage_in_unused_slots(gpu):
    wl = workloads.make_prefill_workload(70, 2, 1, 32, 0, 60, 0, 50, dtype=torch.float32, seed=70)
    for i in range(70):
        ctx = int(wl.context_lens[i])
        if ctx % 16:
            last = wl.block_tables[i, (ctx - 1) // 16].long()
            wl.k_pool[last, :, ctx % 16:, :] = float("nan")
            wl.v_pool[last, :, ctx % 16:, :] = float("nan")
    _check(wl, gpu)


def test_prefill_fp32_non_causal_and_decode_agreement(gpu):
    """Without the causal rule every row sees the whole context; and the last row of a causal chunk
    equals a decode step over the same pools (two kernels, one answer)."""
    from oracle.dense_attention import dense_attention
    wl = workloads.make_prefill_workload(3, 6, 2, 128, 20, 400, 30, 70, dtype=torch.float32, seed=23)
    out, d = _run(wl, gpu, causal=False)
    kp, vp = d.k_pool.cpu(), d.v_pool.cpu()
    refs = []
    for i in range(3):
        lo, hi = int(wl.cu_seqlens_q[i]), int(wl.cu_seqlens_q[i + 1])
        ctx = int(wl.context_lens[i])
        k = oracle_paged.gather_kv(kp, wl.block_tables[i], ctx)
        v = oracle_paged.gather_kv(vp, wl.block_tables[i], ctx)
        refs.append(dense_attention(wl.query[lo:hi][None], k, v, None)[0])
    assert (out - torch.cat(refs)).abs().max().item() <= FP32_TOL
    causal = paged_ops.paged_prefill(d.query, d.k_pool, d.v_pool, d.block_tables, d.context_lens, d.cu_seqlens_q,
                                     d.max_chunk_len)
    last = (d.cu_seqlens_q[1:] - 1).long()
    dec = paged_ops.paged_decode(d.query.index_select(0, last), d.k_pool, d.v_pool, d.block_tables, d.context_lens,
                                 int(wl.context_lens.max()))
    torch.cuda.synchronize()
    assert (dec - causal.index_select(0, last)).abs().max().item() <= 2e-5


def test_prefill_fp32_llama7b_chunk(gpu):
    """One sequence at the benchmark's dims in fp32: 32 heads of 128, a 512-token chunk behind
    2 048 cached tokens (what ran as 512 decode rows per head before this kernel existed)."""
    wl = workloads.make_prefill_workload(1, 32, 32, 128, 2048, 2048, 512, 512, dtype=torch.float32, seed=1)
    _check(wl, gpu)


def test_prefill_fp16(gpu):
    wl = workloads.make_prefill_workload(3, 4, 2, 128, 0, 300, 1, 140, dtype=torch.float16, seed=3)
    _check(wl, gpu)


def test_prefill_ragged_batch_with_empty_chunk(gpu):
    wl = workloads.make_prefill_workload(5, 4, 4, 128, 0, 120, 0, 90, seed=11)
    assert 0 in wl.chunk_lens or True
    _check(wl, gpu)


def test_prefill_garbage_in_unused_slots(gpu):
    wl = workloads.make_prefill_workload(3, 4, 2, 128, 3, 70, 5, 60, seed=13)
    nan = torch.tensor(float("nan"), dtype=torch.bfloat16)
    for i in range(3):
        ctx = int(wl.context_lens[i])
        last = wl.block_tables[i, (ctx - 1) // 16].long()
        used = (ctx - 1) % 16 + 1
        wl.k_pool[last, :, used:, :] = nan
        wl.v_pool[last, :, used:, :] = nan
    _check(wl, gpu)


def test_prefill_equals_decode_for_single_token_chunks(gpu):
    """A 1-token chunk is a decode step: both kernels must agree."""
    wl = workloads.make_prefill_workload(4, 8, 4, 128, 10, 500, 1, 1, seed=17)
    out, d = _run(wl, gpu)
    q = d.query.view(4, 8, 128)
    dec = paged_ops.paged_decode(q, d.k_pool, d.v_pool, d.block_tables, d.context_lens,
                                 int(wl.context_lens.max()))
    torch.cuda.synchronize()
    assert (out.float() - dec.cpu().float()).abs().max().item() <= 4e-3


def test_prefill_non_causal_sees_whole_context(gpu):
    wl = workloads.make_prefill_workload(2, 4, 4, 128, 20, 90, 30, 70, seed=19)
    out, d = _run(wl, gpu, causal=False)
    from oracle.dense_attention import dense_attention
    kp, vp = d.k_pool.cpu(), d.v_pool.cpu()
    refs = []
    for i in range(2):
        lo, hi = int(wl.cu_seqlens_q[i]), int(wl.cu_seqlens_q[i + 1])
        ctx = int(wl.context_lens[i])
        k = oracle_paged.gather_kv(kp, wl.block_tables[i], ctx)
        v = oracle_paged.gather_kv(vp, wl.block_tables[i], ctx)
        refs.append(dense_attention(wl.query[lo:hi][None], k, v, None)[0])
    assert (out.float() - torch.cat(refs).float()).abs().max().item() <= TOL


def test_prefill_scaled_llama7b_slice(gpu):
    """The benchmark shape at reduced batch: 32 heads, head_dim 128, prefix up to 4096, 512-token chunks."""
    wl = workloads.make_prefill_workload(2, 32, 32, 128, 0, 4096, 512, 512, seed=0)
    _check(wl, gpu)


def test_prefill_long_prefix(gpu):
    """A 300-token chunk behind 30 000 cached tokens (470 K/V tiles per workgroup), block size 64."""
    wl = workloads.make_prefill_workload(2, 4, 2, 128, 30000, 30000, 300, 300, block_size=64, seed=31)
    _check(wl, gpu)
