"""The benchmark configurations at FULL size through the C ABI, every sequence
against the CPU oracle at the stated bar (max-abs 2e-2, bf16), plus a reduced
slice of the GQA configuration on its own length range.

Values are drawn on the GPU (host generation of several GB would dominate) and
copied to the host for the oracle, so both sides see the same bits.  The
oracle needs a second or two per configuration."""
import numpy as np
import pytest
import torch

from ironcore_amd import paged_ops, workloads
from oracle import paged as oracle_paged

pytestmark = pytest.mark.gpu

BAR = 2e-2


def _oracle_decode(wl):
    return oracle_paged.paged_decode(wl.query.cpu(), wl.k_pool.cpu(), wl.v_pool.cpu(), wl.block_tables.cpu(),
                                     wl.context_lens.cpu())


def _hold_all_rows(out, ref, what):
    out = out.float().cpu()
    assert torch.isfinite(out).all(), what
    per_seq = (out - ref.float()).abs().amax(dim=1)
    worst = int(per_seq.argmax())
    assert per_seq[worst].item() <= BAR, f"{what}: sequence {worst} max|diff| {per_seq[worst].item()} > {BAR}"
    return per_seq.max().item()


def _decode(wl, **kw):
    out = paged_ops.paged_decode(wl.query, wl.k_pool, wl.v_pool, wl.block_tables, wl.context_lens,
                                 wl.max_context_len, **kw)
    torch.cuda.synchronize()
    return out


def test_decode_scaled_llama70b_slice(gpu):
    """The GQA configuration's head layout (64 query / 8 KV heads) on its own
    length range, ctx uniform in [1024, 8192], at batch 12: rows are cut over
    two to three waves, so the split-K partials and the reduce pass carry 8
    query heads per slot."""
    wl = workloads.make_decode_workload(12, 64, 8, 128, 1024, 8192, seed=70, device=gpu, device_values=True)
    print(f"llama70b slice: contexts {wl.context_lens.tolist()}", flush=True)
    ref = _oracle_decode(wl)
    _hold_all_rows(_decode(wl), ref, "llama70b slice")
    # the split must not matter: one tile per share, and a few long shares
    for mc in (16, 2048):
        _hold_all_rows(_decode(wl, min_chunk_tokens=mc), ref, f"llama70b slice, min_chunk_tokens {mc}")


def test_full_llama7b_decode(gpu):
    wl = workloads.llama7b_decode(device=gpu, seed=0)
    assert (wl.batch, wl.hn, wl.gn) == (64, 32, 32)
    worst = _hold_all_rows(_decode(wl), _oracle_decode(wl), wl.name)
    print(f"{wl.name}: all {wl.batch} sequences, max|diff| {worst:.3e}", flush=True)


def test_full_llama70b_gqa_decode(gpu):
    wl = workloads.llama70b_gqa_decode(device=gpu, seed=0)
    assert (wl.batch, wl.hn, wl.gn) == (128, 64, 8)
    assert int(wl.context_lens.min()) >= 1024 and int(wl.context_lens.max()) <= 8192
    worst = _hold_all_rows(_decode(wl), _oracle_decode(wl), wl.name)
    print(f"{wl.name}: all {wl.batch} sequences, max|diff| {worst:.3e}", flush=True)


def test_full_qwen7b_grpo_decode_with_and_without_cohorts(gpu):
    wl = workloads.qwen7b_grpo_decode(device=gpu, seed=0)
    assert (wl.batch, wl.hn, wl.gn) == (512, 28, 4)
    ref = _oracle_decode(wl)
    plain = _decode(wl)
    worst_plain = _hold_all_rows(plain, ref, wl.name + " (plain)")
    shared = torch.from_numpy(paged_ops.shared_prefix_blocks(
        wl.block_tables.cpu().numpy(), wl.context_lens.cpu().numpy(), wl.block_size, 16)).to(gpu)
    assert int(shared.min()) == 64          # every group aliases its 1024-token prompt
    coh = _decode(wl, cohort_size=16, cohort_shared_blocks=shared)
    worst_coh = _hold_all_rows(coh, ref, wl.name + " (cohorts of 16)")
    print(f"{wl.name}: all {wl.batch} sequences, max|diff| plain {worst_plain:.3e}, cohorts {worst_coh:.3e}",
          flush=True)


def test_full_llama7b_chunked_prefill_and_append(gpu):
    wl = workloads.llama7b_chunked_prefill(device=gpu, seed=0)
    assert len(wl.chunk_lens) == 16 and set(wl.chunk_lens) == {512}
    before_k, before_v = wl.k_pool.clone(), wl.v_pool.clone()
    paged_ops.kv_append(wl.k_new, wl.v_new, wl.k_pool, wl.v_pool, wl.slot_mapping)
    out = paged_ops.paged_prefill(wl.query, wl.k_pool, wl.v_pool, wl.block_tables, wl.context_lens,
                                  wl.cu_seqlens_q, wl.max_chunk_len)
    torch.cuda.synchronize()
    # append, bit for bit: the closed form on the device's own copy of the old pool
    kp, vp = before_k.cpu(), before_v.cpu()
    sm = wl.slot_mapping.cpu()
    kp[sm // 16, :, sm % 16, :] = wl.k_new.cpu()
    vp[sm // 16, :, sm % 16, :] = wl.v_new.cpu()
    assert torch.equal(wl.k_pool.cpu().view(torch.int16), kp.view(torch.int16)), "append K not bit-exact"
    assert torch.equal(wl.v_pool.cpu().view(torch.int16), vp.view(torch.int16)), "append V not bit-exact"
    ref = oracle_paged.paged_prefill(wl.query.cpu(), kp, vp, wl.block_tables.cpu(), wl.context_lens.cpu(),
                                     wl.cu_seqlens_q.cpu())
    diff = (out.float().cpu() - ref.float()).abs().amax(dim=1).view(16, 512).amax(dim=1)
    worst = int(diff.argmax())
    assert diff[worst].item() <= BAR, f"sequence {worst} (prefix {wl.prefix_lens[worst]}): {diff[worst].item()}"
    print(f"{wl.name}: all 16 sequences, max|diff| {diff.max().item():.3e}", flush=True)
