"""Rotary embedding fused into the KV append, through the C ABI, against the
CPU oracle (rotary.py:69-83 restated).  The kernel performs the same fp32
products and sums in the same order and rounds once to the element type, so
the comparison is BIT-EXACT for the rotated query rows and for the pools."""
import pytest
import torch

from ironcore_amd import paged_ops
from ironcore_amd._lib import PagedLibraryError
from oracle import paged as oracle_paged
from oracle import rope as oracle_rope

pytestmark = pytest.mark.gpu

BITS = {torch.bfloat16: torch.int16, torch.float16: torch.int16, torch.float32: torch.int32}


def _case(n, hn, gn, hd, dtype, seed, num_blocks=12, block_size=16, max_pos=300):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(n, hn, hd, generator=g).to(dtype)
    k = torch.randn(n, gn, hd, generator=g).to(dtype)
    v = torch.randn(n, gn, hd, generator=g).to(dtype)
    kp = torch.randn(num_blocks, gn, block_size, hd, generator=g).to(dtype)
    vp = torch.randn(num_blocks, gn, block_size, hd, generator=g).to(dtype)
    slots = torch.randperm(num_blocks * block_size, generator=g)[:n].to(torch.int64)
    pos = torch.randint(0, max_pos, (n,), generator=g, dtype=torch.int32)
    cos, sin = oracle_rope.rope_tables(hd, max_pos)
    return q, k, v, kp, vp, slots, pos, cos, sin


def _expect(q, k, v, kp, vp, slots, pos, cos, sin):
    dtype = q.dtype
    q_rot = oracle_rope.rope_rotate(q, pos, cos, sin).to(dtype)
    k_rot = oracle_rope.rope_rotate(k, pos, cos, sin).to(dtype)
    kp, vp = kp.clone(), vp.clone()
    oracle_paged.kv_append(kp, vp, k_rot, v, slots)
    return q_rot, kp, vp


def _same(a, b):
    return torch.equal(a.cpu().contiguous().view(BITS[a.dtype]), b.contiguous().view(BITS[b.dtype]))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("hn,gn,hd", [(8, 2, 128), (4, 4, 64), (28, 4, 128)])
def test_rotate_and_append_bit_exact(gpu, dtype, hn, gn, hd):
    case = _case(37, hn, gn, hd, dtype, seed=hn + hd)
    want_q, want_kp, want_vp = _expect(*case)
    q, k, v, kp, vp, slots, pos, cos, sin = [t.to(gpu) for t in case]
    paged_ops.rope_kv_append(q, k, v, kp, vp, slots, pos, cos, sin)
    torch.cuda.synchronize()
    assert _same(q, want_q), "rotated query differs"
    assert _same(kp, want_kp), "K pool differs"
    assert _same(vp, want_vp), "V pool differs"


def test_query_only_and_kv_only(gpu):
    case = _case(20, 8, 4, 128, torch.bfloat16, seed=5)
    want_q, want_kp, want_vp = _expect(*case)
    q, k, v, kp, vp, slots, pos, cos, sin = [t.to(gpu) for t in case]
    paged_ops.rope_kv_append(q, None, None, None, None, None, pos, cos, sin)
    torch.cuda.synchronize()
    assert _same(q, want_q) and _same(kp, case[3]) and _same(vp, case[4])
    paged_ops.rope_kv_append(None, k, v, kp, vp, slots, pos, cos, sin)
    torch.cuda.synchronize()
    assert _same(kp, want_kp) and _same(vp, want_vp) and _same(q, want_q)


def test_padding_slots_are_skipped_and_positions_clamped(gpu):
    case = list(_case(16, 4, 2, 64, torch.bfloat16, seed=9, max_pos=40))
    case[5][3] = -1                      # a padding row: nothing is written for it
    case[5][7] = 10 ** 9                 # out of the pool: skipped too
    q, k, v, kp, vp, slots, pos, cos, sin = case
    keep = (slots >= 0) & (slots < 12 * 16)
    k_rot = oracle_rope.rope_rotate(k, pos, cos, sin).to(k.dtype)
    want_kp, want_vp = kp.clone(), vp.clone()
    oracle_paged.kv_append(want_kp, want_vp, k_rot[keep], v[keep], slots[keep])
    pos_bad = pos.clone()
    pos_bad[0], pos_bad[1] = -5, 1000    # clamped to rows 0 and 39
    pos_ok = pos.clone()
    pos_ok[0], pos_ok[1] = 0, 39
    want_q = oracle_rope.rope_rotate(q, pos_ok, cos, sin).to(q.dtype)
    qd = q.to(gpu)
    paged_ops.rope_kv_append(qd, None, None, None, None, None, pos_bad.to(gpu), cos.to(gpu), sin.to(gpu))
    kpd, vpd = kp.to(gpu), vp.to(gpu)
    paged_ops.rope_kv_append(None, k.to(gpu), v.to(gpu), kpd, vpd, slots.to(gpu), pos.to(gpu), cos.to(gpu),
                             sin.to(gpu))
    torch.cuda.synchronize()
    assert _same(qd, want_q) and _same(kpd, want_kp) and _same(vpd, want_vp)


def test_strided_rows_and_token_major_pool(gpu):
    q, k, v, kp, vp, slots, pos, cos, sin = _case(24, 8, 2, 128, torch.bfloat16, seed=11)
    want_q, want_kp, want_vp = _expect(q, k, v, kp, vp, slots, pos, cos, sin)
    # K and V as the two halves of one projection output; pools stored token-major
    kv = torch.cat([k, v], dim=1).to(gpu)                 # [n, 2*gn, hd]
    kd, vd = kv[:, :2], kv[:, 2:]
    kpd = kp.permute(0, 2, 1, 3).contiguous().to(gpu).permute(0, 2, 1, 3)
    vpd = vp.permute(0, 2, 1, 3).contiguous().to(gpu).permute(0, 2, 1, 3)
    qd = q.to(gpu)
    paged_ops.rope_kv_append(qd, kd, vd, kpd, vpd, slots.to(gpu), pos.to(gpu), cos.to(gpu), sin.to(gpu))
    torch.cuda.synchronize()
    assert _same(qd, want_q) and _same(kpd, want_kp) and _same(vpd, want_vp)


def test_position_zero_leaves_rows_unchanged_and_rejects_bad_tables(gpu):
    q, k, v, kp, vp, slots, pos, cos, sin = _case(8, 4, 2, 64, torch.bfloat16, seed=13)
    qd = q.to(gpu)
    paged_ops.rope_kv_append(qd, None, None, None, None, None, torch.zeros(8, dtype=torch.int32, device=gpu),
                             cos.to(gpu), sin.to(gpu))
    torch.cuda.synchronize()
    assert _same(qd, q)
    with pytest.raises(ValueError):
        paged_ops.rope_kv_append(qd, None, None, None, None, None, pos.to(gpu), cos[:, :16].contiguous().to(gpu),
                                 sin[:, :16].contiguous().to(gpu))


def test_rotated_keys_give_relative_position_scores_through_decode(gpu):
    """Keys appended with positions p and a query rotated with position P score
    as a function of P - p only: shifting every position by a constant leaves the
    paged-decode output unchanged (to bf16 rounding of the rotated rows)."""
    g = torch.Generator().manual_seed(21)
    hn, gn, hd, ctx = 8, 2, 128, 50
    cos, sin = oracle_rope.rope_tables(hd, 512)
    k = torch.randn(ctx, gn, hd, generator=g).bfloat16()
    v = torch.randn(ctx, gn, hd, generator=g).bfloat16()
    q = torch.randn(1, hn, hd, generator=g).bfloat16()
    outs = []
    for shift in (0, 100, 333):
        kp = torch.zeros(4, gn, 16, hd, dtype=torch.bfloat16, device=gpu)
        vp = torch.zeros_like(kp)
        slots = torch.arange(ctx, dtype=torch.int64, device=gpu)
        pos = (torch.arange(ctx, dtype=torch.int32) + shift).to(gpu)
        paged_ops.rope_kv_append(None, k.to(gpu), v.to(gpu), kp, vp, slots, pos, cos.to(gpu), sin.to(gpu))
        qd = q.clone().to(gpu)
        paged_ops.rope_kv_append(qd, None, None, None, None, None,
                                 torch.tensor([ctx - 1 + shift], dtype=torch.int32, device=gpu), cos.to(gpu),
                                 sin.to(gpu))
        bt = torch.arange(4, dtype=torch.int32, device=gpu).view(1, 4)
        out = paged_ops.paged_decode(qd, kp, vp, bt, torch.tensor([ctx], dtype=torch.int32, device=gpu), ctx)
        torch.cuda.synchronize()
        outs.append(out.float().cpu())
    assert (outs[0] - outs[1]).abs().max().item() < 3e-2
    assert (outs[0] - outs[2]).abs().max().item() < 3e-2


def test_rotary_module_mirror(gpu):
    """The module mirror: with positions it rotates each token by its own table
    row; without, like the reference (rotary.py:55-64), by the row's BATCH index."""
    from ironcore_amd.layers import RotaryPositionalEmbedding
    rot = RotaryPositionalEmbedding(64, max_seq_len=128, base=10000, scale=1.0, offset=2).to(gpu)
    cos, sin = oracle_rope.rope_tables(64, 128, 10000, 1.0, 2)
    assert torch.equal(rot.cos_emb.cpu(), cos) and torch.equal(rot.sin_emb.cpu(), sin)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(3, 5, 4, 64, generator=g).bfloat16()
    pos = torch.randint(0, 128, (3, 5), generator=g)
    got = rot(x.to(gpu), pos.to(gpu))
    want = oracle_rope.rope_rotate(x.reshape(15, 4, 64), pos.reshape(-1), cos, sin).bfloat16().view(3, 5, 4, 64)
    assert _same(got, want)
    got = rot(x.to(gpu))
    batch_index = torch.arange(3).repeat_interleave(5)
    want = oracle_rope.rope_rotate(x.reshape(15, 4, 64), batch_index, cos, sin).bfloat16().view(3, 5, 4, 64)
    assert _same(got, want)


@pytest.mark.parametrize("seed", range(24))
def test_random_shapes_bit_exact(gpu, seed):
    """Seeded random row counts, head layouts, element types, block sizes and
    padding slots: the rotary append and the plain append, bit for bit."""
    import random
    rng = random.Random(seed)
    dtype = rng.choice([torch.bfloat16, torch.float16, torch.float32])
    hn, gn = rng.choice([(1, 1), (3, 1), (8, 2), (12, 12), (28, 4), (40, 8), (5, 5)])
    hd = rng.choice([64, 128])
    block = rng.choice([16, 32, 64])
    nb = rng.randint(1, 20)
    n = rng.randint(1, nb * block)
    print(f"append case {seed}: {n} rows, {hn}/{gn} heads, hd {hd}, {dtype}, {nb} blocks of {block}", flush=True)
    case = list(_case(n, hn, gn, hd, dtype, seed, num_blocks=nb, block_size=block, max_pos=rng.choice([8, 300, 5000])))
    for i in rng.sample(range(n), rng.randint(0, min(n, 5))):
        case[5][i] = -1                                    # padding rows go nowhere
    want_q, want_kp, want_vp = _expect(*case)
    q, k, v, kp, vp, slots, pos, cos, sin = [t.to(gpu) for t in case]
    plain_k, plain_v = kp.clone(), vp.clone()
    paged_ops.rope_kv_append(q, k, v, kp, vp, slots, pos, cos, sin)
    paged_ops.kv_append(k, v, plain_k, plain_v, slots)
    torch.cuda.synchronize()
    assert _same(q, want_q), "rotated query differs"
    assert _same(kp, want_kp), "K pool differs"
    assert _same(vp, want_vp), "V pool differs"
    want_plain_k, want_plain_v = case[3].clone(), case[4].clone()
    oracle_paged.kv_append(want_plain_k, want_plain_v, case[1], case[2], case[5])
    assert _same(plain_k, want_plain_k) and _same(plain_v, want_plain_v), "plain append differs"
