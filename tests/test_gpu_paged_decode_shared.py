"""Shared-prefix (cohort) paged decode through the C ABI.

The cohort entry point must return what the plain one returns (it only reads
aliased prefix blocks once), so every case is checked twice: against the CPU
oracle (max-abs 2e-2 for bf16/fp16) and against ``ic_paged_decode`` on the
same inputs."""
import numpy as np
import pytest
import torch

from ironcore_amd import paged_ops, workloads
from ironcore_amd._lib import PagedLibraryError
from oracle import paged as oracle_paged

pytestmark = pytest.mark.gpu

TOL = 2e-2


def _shared(wl, cohort_size):
    return paged_ops.shared_prefix_blocks(wl.block_tables.numpy(), wl.context_lens.numpy(), wl.block_size,
                                          cohort_size)


def _run(wl, gpu, cohort_size, shared=None, **kw):
    d = wl.to(gpu)
    if cohort_size > 1:
        if shared is None:
            shared = _shared(wl, cohort_size)
        kw["cohort_shared_blocks"] = torch.from_numpy(np.ascontiguousarray(shared, dtype=np.int32)).to(gpu)
    out = paged_ops.paged_decode(d.query, d.k_pool, d.v_pool, d.block_tables, d.context_lens,
                                 d.max_context_len, cohort_size=cohort_size, **kw)
    torch.cuda.synchronize()
    return out.cpu()


def _check(wl, out, plain):
    # the oracle needs at least one token per sequence; empty ones are checked by the caller
    ctx = wl.context_lens.clamp(min=1)
    ref = oracle_paged.paged_decode(wl.query, wl.k_pool, wl.v_pool, wl.block_tables, ctx)
    ref[wl.context_lens <= 0] = 0
    assert torch.isfinite(out.float()).all()
    diff = (out.float() - ref.float()).abs().max().item()
    assert diff <= TOL, f"vs oracle: max|diff| {diff} ({wl.name})"
    same = (out.float() - plain.float()).abs().max().item()
    assert same <= 4e-3, f"vs plain decode: max|diff| {same} ({wl.name})"


@pytest.mark.parametrize("hn,gn,cohort", [(28, 4, 2), (28, 4, 4), (28, 4, 8), (28, 4, 16), (8, 8, 16), (8, 8, 32),
                                         (16, 2, 2), (16, 2, 4), (16, 2, 8), (6, 2, 5), (6, 2, 3), (32, 2, 2),
                                         (32, 2, 8), (4, 4, 100)])
def test_grpo_groups(gpu, hn, gn, cohort):
    """Groups of samples that alias a 96-token prompt; the cohort size divides,
    equals or straddles the group size."""
    wl = workloads.make_grpo_workload(3, 8, hn, gn, 128, 96, 1, 200, seed=hn + cohort)
    plain = _run(wl, gpu, 1)
    _check(wl, _run(wl, gpu, cohort), plain)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("hd", [64, 128])
def test_dtypes_head_dims(gpu, dtype, hd):
    wl = workloads.make_grpo_workload(4, 4, 8, 2, hd, 64, 1, 90, dtype=dtype, seed=hd)
    plain = _run(wl, gpu, 1)
    _check(wl, _run(wl, gpu, 4), plain)
    _check(wl, _run(wl, gpu, 2), plain)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("hd", [64, 128])
@pytest.mark.parametrize("cohort", [4, 8, 16])
def test_workgroup_wide_cohorts(gpu, dtype, hd, cohort):
    """Cohorts that take 2, 4 and 8 waves (7 heads per KV head: two members per
    wave): the shared tiles go through the LDS ring of a workgroup, in both
    head dims and element types; prompts of 1 to 3 rounds of the ring and a
    ragged last round."""
    wl = workloads.make_grpo_workload(3, 16, 28, 4, hd, 16 * (cohort + 3), 1, 150, dtype=dtype, seed=hd + cohort)
    plain = _run(wl, gpu, 1)
    _check(wl, _run(wl, gpu, cohort), plain)


def test_no_sharing_declared(gpu):
    """cohort_shared_blocks may under-state the sharing: zeros are always valid."""
    wl = workloads.make_grpo_workload(2, 4, 28, 4, 128, 64, 1, 100, seed=1)
    plain = _run(wl, gpu, 1)
    _check(wl, _run(wl, gpu, 2, shared=np.zeros(4, dtype=np.int32)), plain)
    _check(wl, _run(wl, gpu, 2, shared=np.array([1, 0, 4, 2], dtype=np.int32)), plain)


def test_independent_sequences(gpu):
    """Cohorts over sequences that share nothing (the helper reports 0 blocks)."""
    wl = workloads.make_decode_workload(7, 16, 4, 128, 1, 700, seed=3)
    assert _shared(wl, 2).tolist()[:3] == [0, 0, 0]  # (the last cohort has one member)
    plain = _run(wl, gpu, 1)
    _check(wl, _run(wl, gpu, 2), plain)


def test_prefix_is_whole_context(gpu):
    """Right after a fork every member's context is the shared prompt plus the
    one token just appended; with a block-aligned prompt of 64 and suffix 0 or 1
    some members have no private tile at all."""
    wl = workloads.make_grpo_workload(3, 4, 8, 2, 128, 64, 1, 1, seed=8)
    plain = _run(wl, gpu, 1)
    _check(wl, _run(wl, gpu, 4), plain)
    # all members stop exactly at the prefix end: no private tiles anywhere
    wl.context_lens[:] = 64
    wl.max_context_len = 64
    plain = _run(wl, gpu, 1)
    _check(wl, _run(wl, gpu, 4), plain)


def test_ragged_last_cohort_and_empty_member(gpu):
    wl = workloads.make_grpo_workload(1, 7, 8, 4, 128, 48, 1, 120, seed=2)  # 7 sequences, cohorts of 4: 4 + 3
    wl.context_lens[2] = 0  # an empty member kills the sharing of its cohort and yields zeros
    plain = _run(wl, gpu, 1)
    out = _run(wl, gpu, 4)
    _check(wl, out, plain)
    assert torch.count_nonzero(out[2]) == 0


@pytest.mark.parametrize("min_chunk_tokens", [16, 64, 1024, 1 << 20])
def test_split_invariance(gpu, min_chunk_tokens):
    wl = workloads.make_grpo_workload(4, 4, 28, 4, 128, 512, 1, 600, seed=5)
    plain = _run(wl, gpu, 1)
    _check(wl, _run(wl, gpu, 2, min_chunk_tokens=min_chunk_tokens), plain)
    _check(wl, _run(wl, gpu, 4, min_chunk_tokens=min_chunk_tokens), plain)


def test_block_size_64(gpu):
    wl = workloads.make_grpo_workload(3, 4, 8, 2, 128, 128, 1, 300, block_size=64, seed=4)
    plain = _run(wl, gpu, 1)
    _check(wl, _run(wl, gpu, 4), plain)


def test_rejects_too_many_columns_and_fp32(gpu):
    wl = workloads.make_grpo_workload(2, 8, 28, 4, 128, 32, 1, 40, seed=6)
    with pytest.raises(ValueError):
        _run(wl, gpu, 17, shared=np.zeros(1, dtype=np.int32))  # 7 heads: 2 members per wave, 9 waves > 8
    wl17 = workloads.make_grpo_workload(2, 4, 34, 2, 64, 32, 1, 40, seed=6)
    with pytest.raises(ValueError):
        _run(wl17, gpu, 2, shared=np.zeros(4, dtype=np.int32))  # 17 heads per KV head > 16 columns
    wl32 = workloads.make_grpo_workload(2, 4, 8, 4, 64, 32, 1, 40, dtype=torch.float32, seed=6)
    with pytest.raises(PagedLibraryError):
        _run(wl32, gpu, 2)


def test_scaled_grpo_slice(gpu):
    """The GRPO benchmark shape (28 q heads, 4 kv heads, 1024-token prompt) at
    4 prompts x 16 samples, with the cohort the benchmark uses and a narrower one."""
    wl = workloads.make_grpo_workload(4, 16, 28, 4, 128, 1024, 1, 1024, seed=0)
    plain = _run(wl, gpu, 1)
    _check(wl, _run(wl, gpu, 16), plain)
    _check(wl, _run(wl, gpu, 4), plain)


def test_wide_cohorts_of_unequal_prefixes_and_block_64(gpu):
    """Members of a wide cohort alias only the blocks the helper finds equal in
    ALL its rows: cohorts of 16 laid over groups of 4 share nothing, cohorts of
    8 over groups of 16 share everything; 64-token pool blocks (4 tiles each)."""
    wl = workloads.make_grpo_workload(4, 4, 28, 4, 128, 256, 1, 300, block_size=64, seed=11)
    plain = _run(wl, gpu, 1)
    assert _shared(wl, 16).tolist() == [0]
    _check(wl, _run(wl, gpu, 16), plain)
    wl = workloads.make_grpo_workload(2, 16, 28, 4, 128, 256, 1, 300, block_size=64, seed=12)
    assert _shared(wl, 8).tolist() == [4, 4, 4, 4]
    plain = _run(wl, gpu, 1)
    _check(wl, _run(wl, gpu, 8), plain)


def test_forked_samples_through_the_layer(gpu):
    """A prompt prefilled once, forked into samples, then decoded through the
    attention layer with and without cohorts: same output."""
    from types import SimpleNamespace
    from ironcore_amd import config as ic_config
    from ironcore_amd.kv_cache import PagedKVCache
    from ironcore_amd.layers import Attention

    hn, gn, hd, n_samples = 28, 4, 128, 6
    cfg = ic_config.MainConfig(model=ic_config.ModelConfig(
        d_model=hn * hd, num_attention_heads=hn, num_attention_groups=gn, head_dim=hd, dropout_attn=0.0,
        precision="bf16"), trainer=ic_config.TrainerConfig(use_flash_attn=False))
    attn = Attention(cfg).to(gpu).eval()
    cache = PagedKVCache(1, 64, 16, gn, hd, torch.bfloat16, gpu)
    g = torch.Generator().manual_seed(3)
    root = cache.add_sequence()
    sq = 70
    q = torch.randn(1, sq, hn, hd, generator=g).bfloat16().to(gpu)
    k = torch.randn(1, sq, gn, hd, generator=g).bfloat16().to(gpu)
    v = torch.randn(1, sq, gn, hd, generator=g).bfloat16().to(gpu)
    attn(q, k, v, None, kv_cache=cache.layer(0), attn_metadata=cache.prepare([root], sq))
    ids = [root] + [cache.fork(root) for _ in range(n_samples - 1)]
    for step in range(3):
        q = torch.randn(n_samples, 1, hn, hd, generator=g).bfloat16().to(gpu)
        k = torch.randn(n_samples, 1, gn, hd, generator=g).bfloat16().to(gpu)
        v = torch.randn(n_samples, 1, gn, hd, generator=g).bfloat16().to(gpu)
        meta = cache.prepare(ids, 1, cohort_size=4)
        assert meta.cohort_size == 4 and meta.cohort_shared_blocks.tolist()[0] == 4
        got = attn(q, k, v, None, kv_cache=cache.layer(0), attn_metadata=meta)
        plain_meta = SimpleNamespace(**{**meta.__dict__, "cohort_size": 1, "cohort_shared_blocks": None,
                                        "slot_mapping": torch.full_like(meta.slot_mapping, -1)})
        want = attn(q, k, v, None, kv_cache=cache.layer(0), attn_metadata=plain_meta)
        torch.cuda.synchronize()
        assert (got.float() - want.float()).abs().max().item() <= 4e-3, f"step {step}"
