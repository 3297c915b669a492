"""The masked entry points on real block tables (ic_paged_prefill_masked,
ic_paged_decode_masked through paged_ops): many blocks per sequence, randomly
permuted, GQA, per-head and shared masks, rows with no visible key, a mask
narrower than the context.  Against the oracle: the reference's dense
attention with masked_fill(mask == 0, finfo.min) (attention.py:115-117) on the
gathered rows."""
import pytest
import torch

from ironcore_amd import paged_ops, workloads
from oracle import paged as oracle_paged
from oracle.dense_attention import dense_attention
from parity_bars import hold

pytestmark = pytest.mark.gpu


def _prefill_oracle(wl, kp, vp, mask, dtype=None):
    """mask: bool [n_seqs or 1, hn or 1, max_chunk, keys]; keys past its last dimension are hidden."""
    outs = []
    for i in range(wl.context_lens.numel()):
        lo, hi = int(wl.cu_seqlens_q[i]), int(wl.cu_seqlens_q[i + 1])
        if hi == lo:
            continue
        ctx = int(wl.context_lens[i])
        k = oracle_paged.gather_kv(kp, wl.block_tables[i], ctx)
        v = oracle_paged.gather_kv(vp, wl.block_tables[i], ctx)
        q = wl.query[lo:hi][None]
        m = mask[i if mask.shape[0] > 1 else 0][:, :hi - lo, :ctx]          # [mh, C, <= ctx]
        if m.shape[-1] < ctx:
            m = torch.cat([m, torch.zeros(*m.shape[:-1], ctx - m.shape[-1], dtype=m.dtype)], dim=-1)
        if dtype is not None:
            q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
        outs.append(dense_attention(q, k, v, m[None])[0])
    return torch.cat(outs)


@pytest.mark.parametrize("block,hd", [(16, 128), (64, 64), (16, 32), (48, 128)])
@pytest.mark.parametrize("per_head,per_seq", [(True, True), (False, True), (False, False)])
def test_masked_prefill_on_block_tables(gpu, block, hd, per_head, per_seq):
    hn, gn, n_seqs = 6, 2, 3
    wl = workloads.make_prefill_workload(n_seqs, hn, gn, hd, 30, 400, 20, 150, block_size=block, seed=block + hd)
    g = torch.Generator().manual_seed(block * 7 + hd)
    keys = int(wl.context_lens.max())
    mask = torch.rand(n_seqs if per_seq else 1, hn if per_head else 1, wl.max_chunk_len, keys, generator=g) < 0.7
    mask[..., 0] = True
    mask[0, 0, 3] = False                       # one query row (of every head that shares it) sees nothing
    d = wl.to(gpu)
    paged_ops.kv_append(d.k_new, d.v_new, d.k_pool, d.v_pool, d.slot_mapping)
    out = paged_ops.paged_prefill(d.query, d.k_pool, d.v_pool, d.block_tables, d.context_lens, d.cu_seqlens_q,
                                  d.max_chunk_len, mask=mask.to(torch.uint8).to(gpu))
    torch.cuda.synchronize()
    kp, vp = d.k_pool.cpu(), d.v_pool.cpu()
    ref = _prefill_oracle(wl, kp, vp, mask)
    truth = _prefill_oracle(wl, kp, vp, mask, torch.float64)
    fewest = 1 << 30                              # fewest keys any query row sees (a row that sees none sees all)
    for i, c in enumerate(wl.chunk_lens):
        ctx = int(wl.context_lens[i])
        if c > 0:
            per_row = mask[i if per_seq else 0][:, :c, :ctx].sum(-1)
            fewest = min(fewest, int(torch.where(per_row == 0, torch.full_like(per_row, ctx), per_row).min()))
    hold(out, ref, truth, torch.bfloat16, fewest, f"masked prefill block {block} hd {hd}")
    # the fully hidden row averages V over its whole context (finite fill value)
    ctx0 = int(wl.context_lens[0])
    v0 = oracle_paged.gather_kv(vp, wl.block_tables[0], ctx0)[0].float().mean(dim=0)       # [gn, hd]
    want = v0[0]
    assert (out[3, :hd].cpu().float() - want).abs().max().item() <= 2e-2


def test_masked_prefill_mask_narrower_than_the_context(gpu):
    """Keys past the mask's last dimension are hidden, and nothing is read there."""
    hn, gn, hd = 4, 4, 64
    wl = workloads.make_prefill_workload(2, hn, gn, hd, 100, 200, 40, 60, seed=5)
    keys = int(wl.context_lens.min()) - 30
    g = torch.Generator().manual_seed(6)
    mask = torch.rand(1, 1, wl.max_chunk_len, keys, generator=g) < 0.8
    mask[..., 0] = True
    d = wl.to(gpu)
    paged_ops.kv_append(d.k_new, d.v_new, d.k_pool, d.v_pool, d.slot_mapping)
    out = paged_ops.paged_prefill(d.query, d.k_pool, d.v_pool, d.block_tables, d.context_lens, d.cu_seqlens_q,
                                  d.max_chunk_len, mask=mask.to(torch.uint8).to(gpu))
    torch.cuda.synchronize()
    ref = _prefill_oracle(wl, d.k_pool.cpu(), d.v_pool.cpu(), mask)
    assert (out.cpu().float() - ref.float()).abs().max().item() <= 2e-2


@pytest.mark.parametrize("hn,gn,hd", [(8, 2, 128), (6, 6, 64), (4, 1, 32)])
@pytest.mark.parametrize("per_head", [True, False])
def test_masked_decode_on_block_tables(gpu, hn, gn, hd, per_head):
    """fp32 key-masked decode on block-16 pools with GQA."""
    b = 5
    wl = workloads.make_decode_workload(b, hn, gn, hd, 1, 700, dtype=torch.float32, seed=hn + hd)
    g = torch.Generator().manual_seed(hn)
    key_mask = torch.rand(b, hn if per_head else 1, wl.max_context_len, generator=g) < 0.6
    key_mask[..., 0] = True
    key_mask[1] = False                          # a sequence whose query sees nothing: the mean of V
    d = wl.to(gpu)
    out = paged_ops.paged_decode(d.query, d.k_pool, d.v_pool, d.block_tables, d.context_lens, d.max_context_len,
                                 key_mask=key_mask.to(torch.uint8).to(gpu))
    torch.cuda.synchronize()
    refs = []
    for i in range(b):
        ctx = int(wl.context_lens[i])
        k = oracle_paged.gather_kv(wl.k_pool, wl.block_tables[i], ctx)
        v = oracle_paged.gather_kv(wl.v_pool, wl.block_tables[i], ctx)
        m = key_mask[i][:, None, :ctx][None]      # [1, mh, 1, ctx]
        refs.append(dense_attention(wl.query[i][None, None], k, v, m)[0, 0])
    assert (out.cpu() - torch.stack(refs)).abs().max().item() <= 1e-4
    mean_v = oracle_paged.gather_kv(wl.v_pool, wl.block_tables[1], int(wl.context_lens[1]))[0].mean(dim=0)
    assert (out[1].cpu().view(hn, hd) - mean_v.repeat_interleave(hn // gn, dim=0)).abs().max().item() <= 1e-4


def test_decode_batches_of_changing_size_ask_the_runtime_once(gpu):
    """A serving loop whose batch size changes from step to step (3, 9, 3, 17, 9
    sequences): the launcher keeps the runtime's occupancy answers per kernel
    variant and LDS size class for the whole process, so repeating the shapes
    asks nothing; a second host thread then captures a decode into a graph
    (where a runtime query would be an error) and its replay equals the eager
    result."""
    import threading
    from ironcore_amd import _lib
    lib = _lib.load()
    wls = {n: workloads.make_decode_workload(n, 8, 2, 128, 40, 900, seed=n).to(gpu) for n in (3, 9, 17)}
    outs = {}

    def run(n):
        d = wls[n]
        return paged_ops.paged_decode(d.query, d.k_pool, d.v_pool, d.block_tables, d.context_lens, d.max_context_len)

    for n in (3, 9, 3, 17, 9):
        outs[n] = run(n)
    torch.cuda.synchronize()
    asked = lib.ic_decode_occupancy_queries()
    for n in (3, 9, 3, 17, 9):
        again = run(n)
        assert torch.equal(again, outs[n])
    torch.cuda.synchronize()
    assert lib.ic_decode_occupancy_queries() == asked, "a repeated shape asked the runtime again"

    result = {}

    def capture_on_another_thread():
        try:
            d = wls[9]
            out = torch.empty_like(outs[9])
            stream = torch.cuda.Stream(device=gpu)
            with torch.cuda.stream(stream):
                paged_ops.paged_decode(d.query, d.k_pool, d.v_pool, d.block_tables, d.context_lens,
                                       d.max_context_len, out=out)      # workspace of this stream, before the capture
                stream.synchronize()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=stream):
                    paged_ops.paged_decode(d.query, d.k_pool, d.v_pool, d.block_tables, d.context_lens,
                                           d.max_context_len, out=out)
                for _ in range(3):
                    out.zero_()
                    stream.synchronize()
                    graph.replay()
                    stream.synchronize()
                    assert torch.equal(out, outs[9])
            result["ok"] = True
        except Exception as exc:                                          # noqa: BLE001 (reported below)
            result["error"] = exc

    t = threading.Thread(target=capture_on_another_thread)
    t.start()
    t.join()
    assert result.get("ok"), result.get("error")
    assert lib.ic_decode_occupancy_queries() == asked
