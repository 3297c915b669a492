"""Pins the paged drivers of the oracle (oracle/paged.py): the block-table
gather, the append closed form and the chunked-prefill mask, by properties any
correct block KV cache must have."""
import pytest
import torch

from ironcore_amd import workloads
from oracle import paged as oracle_paged
from oracle.dense_attention import causal_offset_mask, dense_attention


def _contiguous_rows(wl, i):
    """Sequence i's K/V rows gathered by plain Python indexing."""
    ctx = int(wl.context_lens[i])
    ks, vs = [], []
    for p in range(ctx):
        blk = int(wl.block_tables[i, p // wl.block_size])
        ks.append(wl.k_pool[blk, :, p % wl.block_size, :])
        vs.append(wl.v_pool[blk, :, p % wl.block_size, :])
    return torch.stack(ks)[None], torch.stack(vs)[None]


def test_gather_follows_block_table():
    wl = workloads.make_decode_workload(3, 4, 2, 8, 1, 50, dtype=torch.float32, seed=1)
    for i in range(3):
        k, v = _contiguous_rows(wl, i)
        ctx = int(wl.context_lens[i])
        assert torch.equal(oracle_paged.gather_kv(wl.k_pool, wl.block_tables[i], ctx), k)
        assert torch.equal(oracle_paged.gather_kv(wl.v_pool, wl.block_tables[i], ctx), v)


def test_decode_equals_dense_on_contiguous_rows():
    wl = workloads.make_decode_workload(3, 6, 2, 16, 1, 70, dtype=torch.float32, seed=2)
    out = oracle_paged.paged_decode(wl.query, wl.k_pool, wl.v_pool, wl.block_tables, wl.context_lens)
    for i in range(3):
        k, v = _contiguous_rows(wl, i)
        want = dense_attention(wl.query[i][None, None], k, v)[0, 0]
        assert torch.equal(out[i], want)


def test_decode_invariant_under_block_permutation():
    wl = workloads.make_decode_workload(4, 4, 4, 8, 5, 90, dtype=torch.float32, seed=3)
    out1 = oracle_paged.paged_decode(wl.query, wl.k_pool, wl.v_pool, wl.block_tables, wl.context_lens)
    nb = wl.k_pool.shape[0]
    perm = torch.randperm(nb, generator=torch.Generator().manual_seed(0))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(nb)
    out2 = oracle_paged.paged_decode(wl.query, wl.k_pool[perm], wl.v_pool[perm],
                                     inv[wl.block_tables.long()].to(torch.int32), wl.context_lens)
    assert torch.equal(out1, out2)


def test_aliased_prefix_equals_duplicated_blocks():
    wl = workloads.make_grpo_workload(2, 3, 4, 2, 8, 32, 1, 40, dtype=torch.float32, seed=4)
    out = oracle_paged.paged_decode(wl.query, wl.k_pool, wl.v_pool, wl.block_tables, wl.context_lens)
    # physically duplicate the shared prefix blocks of every sequence
    nb = wl.k_pool.shape[0]
    pre = 32 // 16
    extra_k, extra_v, tables = [], [], wl.block_tables.clone()
    for i in range(wl.batch):
        for j in range(pre):
            extra_k.append(wl.k_pool[tables[i, j].long()])
            extra_v.append(wl.v_pool[tables[i, j].long()])
            tables[i, j] = nb + len(extra_k) - 1
    kp = torch.cat([wl.k_pool, torch.stack(extra_k)])
    vp = torch.cat([wl.v_pool, torch.stack(extra_v)])
    assert torch.equal(out, oracle_paged.paged_decode(wl.query, kp, vp, tables, wl.context_lens))


def test_append_closed_form_sentinel_idempotent():
    nb, gn, bs, hd, n = 5, 3, 16, 8, 20
    g = torch.Generator().manual_seed(5)
    k_new, v_new = torch.randn(n, gn, hd, generator=g), torch.randn(n, gn, hd, generator=g)
    slots = torch.randperm(nb * bs, generator=g)[:n]
    slots[4] = -1
    kp = torch.full((nb, gn, bs, hd), 7.25)
    vp = torch.full((nb, gn, bs, hd), -3.5)
    oracle_paged.kv_append(kp, vp, k_new, v_new, slots)
    # closed form: flat token-slot view + index_copy_
    keep = slots >= 0
    want_k = torch.full((nb, gn, bs, hd), 7.25).permute(0, 2, 1, 3).reshape(nb * bs, gn, hd).clone()
    want_k.index_copy_(0, slots[keep], k_new[keep])
    assert torch.equal(kp.permute(0, 2, 1, 3).reshape(nb * bs, gn, hd), want_k)
    touched = torch.zeros(nb * bs, dtype=torch.bool)
    touched[slots[keep]] = True
    assert (vp.permute(0, 2, 1, 3).reshape(nb * bs, gn, hd)[~touched] == -3.5).all()
    before = kp.clone()
    oracle_paged.kv_append(kp, vp, k_new, v_new, slots)
    assert torch.equal(kp, before)


@pytest.mark.parametrize("prefix,chunk", [(0, 7), (5, 1), (19, 13), (32, 16)])
def test_chunked_prefill_equals_rows_of_full_causal_pass(prefix, chunk):
    """Rows [P, P+C) of one causal pass over P+C tokens == prefill of the chunk
    against a cache holding all P+C rows."""
    hn, gn, hd, bs = 4, 2, 8, 16
    total = prefix + chunk
    g = torch.Generator().manual_seed(prefix * 100 + chunk)
    q_all = torch.randn(1, total, hn, hd, generator=g)
    k_all = torch.randn(1, total, gn, hd, generator=g)
    v_all = torch.randn(1, total, gn, hd, generator=g)
    full = dense_attention(q_all, k_all, v_all, causal_offset_mask(total, total))[0]
    nblk = (total + bs - 1) // bs
    order = torch.randperm(nblk + 2, generator=g)[:nblk]
    kp = torch.zeros(nblk + 2, gn, bs, hd)
    vp = torch.zeros(nblk + 2, gn, bs, hd)
    slots = torch.tensor([int(order[p // bs]) * bs + p % bs for p in range(total)])
    oracle_paged.kv_append(kp, vp, k_all[0], v_all[0], slots)
    out = oracle_paged.paged_prefill(q_all[0, prefix:], kp, vp, order.to(torch.int32)[None],
                                     torch.tensor([total], dtype=torch.int32),
                                     torch.tensor([0, chunk], dtype=torch.int32))
    torch.testing.assert_close(out, full[prefix:], rtol=0, atol=2e-6)


def test_prefill_ragged_batch_and_empty_chunk():
    hn, gn, hd, bs = 2, 2, 4, 16
    g = torch.Generator().manual_seed(9)
    chunks, prefixes = [3, 0, 5], [4, 9, 0]
    tables, ctxs, qs, want = [], [], [], []
    kp = torch.randn(8, gn, bs, hd, generator=g)
    vp = torch.randn(8, gn, bs, hd, generator=g)
    nxt = 0
    for c, pfx in zip(chunks, prefixes):
        total = c + pfx
        nblk = max(1, (total + bs - 1) // bs)
        row = list(range(nxt, nxt + nblk))
        nxt += nblk
        tables.append(row + [0] * (2 - len(row)))
        ctxs.append(total)
        q = torch.randn(c, hn, hd, generator=g)
        qs.append(q)
        if c:
            k = oracle_paged.gather_kv(kp, torch.tensor(row), total)
            v = oracle_paged.gather_kv(vp, torch.tensor(row), total)
            want.append(dense_attention(q[None], k, v, causal_offset_mask(c, total))[0])
    cu = torch.tensor([0, 3, 3, 8], dtype=torch.int32)
    out = oracle_paged.paged_prefill(torch.cat(qs), kp, vp, torch.tensor(tables, dtype=torch.int32),
                                     torch.tensor(ctxs, dtype=torch.int32), cu)
    assert torch.equal(out, torch.cat(want))
