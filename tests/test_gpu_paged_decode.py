"""Paged decode through the C ABI against the CPU oracle (the reference's
dense attention on the gathered rows).  Tolerance: max-abs 2e-2 in bf16/fp16
(the bound the target states), 1e-4 in fp32."""
import pytest
import torch

from ironcore_amd import paged_ops, workloads
from oracle import paged as oracle_paged

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: 2e-2, torch.float16: 2e-2, torch.float32: 1e-4}


def _run(wl, gpu, **kw):
    d = wl.to(gpu)
    out = paged_ops.paged_decode(d.query, d.k_pool, d.v_pool, d.block_tables, d.context_lens,
                                 d.max_context_len, **kw)
    torch.cuda.synchronize()
    return out.cpu()


def _oracle(wl):
    return oracle_paged.paged_decode(wl.query, wl.k_pool, wl.v_pool, wl.block_tables, wl.context_lens)


def _check(wl, out, tol=None):
    ref = _oracle(wl)
    tol = tol or TOL[wl.query.dtype]
    diff = (out.float() - ref.float()).abs().max().item()
    assert torch.isfinite(out.float()).all()
    assert diff <= tol, f"max|diff| {diff} > {tol} ({wl.name})"
    return diff


@pytest.mark.parametrize("hn,gn", [(32, 32), (64, 8), (28, 4), (8, 4), (12, 4), (5, 1), (6, 1), (24, 1)])
def test_decode_group_sizes_bf16(gpu, hn, gn):
    wl = workloads.make_decode_workload(6, hn, gn, 128, 1, 1300, seed=hn * 100 + gn)
    _check(wl, _run(wl, gpu))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("hd", [32, 64, 128])
def test_decode_dtypes_head_dims(gpu, dtype, hd):
    wl = workloads.make_decode_workload(5, 8, 4, hd, 1, 900, dtype=dtype, seed=hd)
    _check(wl, _run(wl, gpu))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("hn,gn", [(8, 8), (8, 1), (7, 1), (24, 2)])
def test_decode_head_dim_32_group_sizes(gpu, dtype, hn, gn):
    """Head dimension 32 (the smallest the reference's own sweep uses,
    tests/test_attention.py:352-379) over MHA, MQA, an odd group and a group
    wider than one wave's columns; contexts long enough for split-K partials."""
    wl = workloads.make_decode_workload(7, hn, gn, 32, 1, 2600, dtype=dtype, seed=hn * 10 + gn)
    out = _run(wl, gpu)
    _check(wl, out)
    one = _run(wl, gpu, min_chunk_tokens=1 << 20)          # one wave walks everything: no partials
    assert (out.float() - one.float()).abs().max().item() <= (4e-3 if dtype != torch.float32 else 1e-5)


def test_unsupported_head_dims_are_named_before_the_c_call(gpu):
    """A head dimension without a kernel is refused in Python, with the list of
    those that have one, not by an error code from the library."""
    kp = torch.zeros(2, 1, 16, 96, dtype=torch.bfloat16, device=gpu)
    tables, lens = torch.zeros(1, 1, dtype=torch.int32, device=gpu), torch.ones(1, dtype=torch.int32, device=gpu)
    q = torch.zeros(1, 1, 96, dtype=torch.bfloat16, device=gpu)
    with pytest.raises(ValueError, match=r"\(32, 64, 128\)"):
        paged_ops.paged_decode(q, kp, kp, tables, lens, 1)
    with pytest.raises(ValueError, match=r"\(32, 64, 128\)"):
        paged_ops.paged_prefill(q, kp, kp, tables, lens, torch.tensor([0, 1], dtype=torch.int32, device=gpu), 1)


@pytest.mark.parametrize("ctx", [1, 2, 15, 16, 17, 31, 32, 33, 511, 512, 513, 1024, 1025])
def test_decode_boundary_lengths(gpu, ctx):
    wl = workloads.make_decode_workload(3, 4, 2, 128, ctx, ctx, seed=ctx)
    _check(wl, _run(wl, gpu))


def test_decode_ctx1_returns_value_row(gpu):
    """One cached token: softmax is 1, so the output is that token's V row, bit for bit."""
    wl = workloads.make_decode_workload(4, 8, 2, 128, 1, 1, seed=11)
    out = _run(wl, gpu)
    for i in range(4):
        v = wl.v_pool[wl.block_tables[i, 0].long(), :, 0, :]          # [gn, hd]
        want = v.repeat_interleave(4, dim=0).reshape(-1)
        assert torch.equal(out[i].view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("min_chunk_tokens", [16, 48, 64, 256, 1024, 4096, 1 << 20])
def test_decode_split_invariance(gpu, min_chunk_tokens):
    """The result does not depend on where the split-K shares are cut; with the
    largest value one wave walks the whole batch."""
    wl = workloads.make_decode_workload(4, 8, 8, 128, 900, 2100, seed=5)
    out = _run(wl, gpu, min_chunk_tokens=min_chunk_tokens)
    _check(wl, out)
    base = _run(wl, gpu, min_chunk_tokens=4096)
    assert (out.float() - base.float()).abs().max().item() <= 4e-3


def test_decode_garbage_in_unused_slots(gpu):
    """NaN/Inf bit patterns beyond the context length and in unused blocks must not leak."""
    wl = workloads.make_decode_workload(4, 8, 4, 128, 5, 200, seed=9, extra_blocks=3)
    ref = _oracle(wl)
    nan = torch.tensor(float("nan"), dtype=torch.bfloat16)
    for i in range(4):
        ctx = int(wl.context_lens[i])
        last = wl.block_tables[i, (ctx - 1) // 16].long()
        used = (ctx - 1) % 16 + 1
        wl.k_pool[last, :, used:, :] = nan
        wl.v_pool[last, :, used:, :] = nan
    out = _run(wl, gpu)
    assert torch.isfinite(out.float()).all()
    assert (out.float() - ref.float()).abs().max().item() <= 2e-2


def test_decode_block_permutation_invariance(gpu):
    wl = workloads.make_decode_workload(4, 8, 4, 128, 100, 700, seed=21)
    out1 = _run(wl, gpu)
    nb = wl.k_pool.shape[0]
    perm = torch.randperm(nb, generator=torch.Generator().manual_seed(1))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(nb)
    wl2 = workloads.DecodeWorkload(**{**wl.__dict__})
    wl2.k_pool = wl.k_pool[perm]
    wl2.v_pool = wl.v_pool[perm]
    wl2.block_tables = inv[wl.block_tables.long()].to(torch.int32)
    out2 = _run(wl2, gpu)
    assert torch.equal(out1.view(torch.int16), out2.view(torch.int16))


def test_decode_grpo_shared_prefix(gpu):
    wl = workloads.make_grpo_workload(3, 4, 28, 4, 128, 128, 1, 200, seed=2)
    _check(wl, _run(wl, gpu))


def test_decode_empty_sequence_and_batch(gpu):
    wl = workloads.make_decode_workload(3, 4, 4, 128, 10, 40, seed=4)
    wl.context_lens[1] = 0
    out = _run(wl, gpu)
    assert torch.count_nonzero(out[1]) == 0
    ref = _oracle(workloads.DecodeWorkload(**{**wl.__dict__, "context_lens": wl.context_lens.clamp(min=1)}))
    assert (out[0].float() - ref[0].float()).abs().max().item() <= 2e-2
    assert (out[2].float() - ref[2].float()).abs().max().item() <= 2e-2


def test_decode_scaled_llama7b_slice(gpu):
    """The headline shape at reduced batch: Llama-7B heads, contexts in [512, 4096]."""
    wl = workloads.make_decode_workload(4, 32, 32, 128, 512, 4096, seed=0)
    _check(wl, _run(wl, gpu))


@pytest.mark.parametrize("batch", [257, 700, 1100])
def test_decode_many_short_sequences(gpu, batch):
    """Batches of more than 256 and of more than 1024 sequences (the prologue
    scans the per-sequence tile counts 256 rows at a time, and keeps them in
    registers only up to 1024 rows), with empty sequences sprinkled in."""
    wl = workloads.make_decode_workload(batch, 4, 2, 64, 1, 70, seed=batch)
    wl.context_lens[::97] = 0
    out = _run(wl, gpu)
    ctx = wl.context_lens.clamp(min=1)
    ref = oracle_paged.paged_decode(wl.query, wl.k_pool, wl.v_pool, wl.block_tables, ctx)
    ref[wl.context_lens <= 0] = 0
    assert torch.isfinite(out.float()).all()
    assert (out.float() - ref.float()).abs().max().item() <= TOL[wl.query.dtype]


def test_decode_step_in_a_captured_graph_and_on_two_streams(gpu):
    """The entry points allocate nothing and only enqueue kernels, so a step
    (append + decode) can be captured in a graph; every replay, interleaved
    with eager work and synchronisations, must equal the eager result.  Two
    streams running different batches at once must not disturb each other
    (each stream has its own split-K scratch)."""
    wl = workloads.make_decode_workload(9, 16, 4, 128, 300, 900, seed=31).to(gpu)
    last = wl.context_lens.long() - 1
    slots = wl.block_tables.long().gather(1, (last // 16).unsqueeze(1)).squeeze(1) * 16 + last % 16
    g = torch.Generator(device=gpu).manual_seed(5)
    k_new = torch.randn(9, 4, 128, generator=g, device=gpu).bfloat16()
    v_new = torch.randn(9, 4, 128, generator=g, device=gpu).bfloat16()
    out = torch.empty(9, 16 * 128, dtype=torch.bfloat16, device=gpu)

    def step():
        paged_ops.kv_append(k_new, v_new, wl.k_pool, wl.v_pool, slots)
        paged_ops.paged_decode(wl.query, wl.k_pool, wl.v_pool, wl.block_tables, wl.context_lens,
                               wl.max_context_len, out=out)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                                   # warm-up on the capture stream: sizes its scratch
    torch.cuda.current_stream().wait_stream(side)
    step()
    torch.cuda.synchronize()
    want = out.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        step()
    for i in range(4):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {i}"
        step()                                   # eager work between replays
        torch.cuda.synchronize()
        assert torch.equal(out, want)
    # two streams, two batches, launched back to back
    wl2 = workloads.make_decode_workload(7, 16, 4, 128, 200, 1200, seed=32).to(gpu)
    ref1 = paged_ops.paged_decode(wl.query, wl.k_pool, wl.v_pool, wl.block_tables, wl.context_lens, wl.max_context_len)
    ref2 = paged_ops.paged_decode(wl2.query, wl2.k_pool, wl2.v_pool, wl2.block_tables, wl2.context_lens,
                                  wl2.max_context_len)
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    for _ in range(5):
        with torch.cuda.stream(s1):
            o1 = paged_ops.paged_decode(wl.query, wl.k_pool, wl.v_pool, wl.block_tables, wl.context_lens,
                                        wl.max_context_len)
        with torch.cuda.stream(s2):
            o2 = paged_ops.paged_decode(wl2.query, wl2.k_pool, wl2.v_pool, wl2.block_tables, wl2.context_lens,
                                        wl2.max_context_len)
    torch.cuda.synchronize()
    assert torch.equal(o1, ref1) and torch.equal(o2, ref2)


def test_decode_batch_beyond_the_lds_plan(gpu):
    """More sequences than the row bookkeeping a workgroup keeps in LDS has room
    for (about 12 000): the kernel variant in which every wave scans the rows
    itself, plain and with shared-prefix cohorts."""
    n = 13000
    wl = workloads.make_decode_workload(n, 4, 2, 64, 1, 40, seed=21)
    out = _run(wl, gpu)
    _check(wl, out)
    shared = torch.from_numpy(paged_ops.shared_prefix_blocks(wl.block_tables.numpy(), wl.context_lens.numpy(),
                                                             wl.block_size, 16)).to(gpu)
    d = wl.to(gpu)
    coh = paged_ops.paged_decode(d.query, d.k_pool, d.v_pool, d.block_tables, d.context_lens, d.max_context_len,
                                 cohort_size=16, cohort_shared_blocks=shared)
    torch.cuda.synchronize()
    _check(wl, coh.cpu())
    # the two variants cut the rows at different tiles and merge in different orders: one step of
    # bf16 at the value's magnitude
    step = torch.maximum(torch.full_like(out.float(), 4e-3), out.float().abs() / 128)
    assert ((coh.cpu().float() - out.float()).abs() - step).max().item() <= 0


@pytest.mark.parametrize("hn,gn,dtype", [(8, 2, torch.bfloat16), (4, 4, torch.float16), (2, 1, torch.float32)])
def test_decode_long_contexts(gpu, hn, gn, dtype):
    """Tens of thousands of tokens per sequence: a wave's share spans many of
    its 256-tile windows and a sequence is cut over hundreds of waves."""
    wl = workloads.make_decode_workload(3, hn, gn, 128, 30000, 70000, dtype=dtype, seed=21)
    _check(wl, _run(wl, gpu))
    _check(wl, _run(wl, gpu, min_chunk_tokens=16384))     # few, long shares: many windows per share
