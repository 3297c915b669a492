"""KV append through the C ABI: bit-exact against the oracle's closed form."""
import pytest
import torch

from ironcore_amd import paged_ops
from oracle import paged as oracle_paged

pytestmark = pytest.mark.gpu


def _case(n, gn, hd, nb, bs, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    if dtype == torch.float32:
        k_new = torch.randn(n, gn, hd, generator=g)
        v_new = torch.randn(n, gn, hd, generator=g)
    else:
        # every bit pattern, NaNs included: the copy must not touch them
        k_new = torch.randint(-32768, 32767, (n, gn, hd), generator=g, dtype=torch.int16).view(dtype)
        v_new = torch.randint(-32768, 32767, (n, gn, hd), generator=g, dtype=torch.int16).view(dtype)
    slots = torch.randperm(nb * bs, generator=g)[:n].to(torch.int64)
    return k_new, v_new, slots


def _bits(t):
    return t.view(torch.int32 if t.element_size() == 4 else torch.int16)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("n,gn,hd,nb", [(1, 1, 64, 3), (37, 4, 128, 9), (300, 32, 128, 40), (64, 12, 64, 8)])
def test_append_bit_exact(gpu, dtype, n, gn, hd, nb):
    bs = 16
    k_new, v_new, slots = _case(n, gn, hd, nb, bs, dtype, seed=n)
    sentinel = 0x5A5A if dtype != torch.float32 else 0x5A5A5A5A
    kp = torch.full((nb, gn, bs, hd), sentinel, dtype=_bits(k_new).dtype).view(dtype)
    vp = kp.clone()
    kp_ref, vp_ref = kp.clone(), vp.clone()
    oracle_paged.kv_append(_bits(kp_ref), _bits(vp_ref), _bits(k_new), _bits(v_new), slots)

    kp_d, vp_d = kp.to(gpu), vp.to(gpu)
    paged_ops.kv_append(k_new.to(gpu), v_new.to(gpu), kp_d, vp_d, slots.to(gpu))
    torch.cuda.synchronize()
    assert torch.equal(_bits(kp_d.cpu()), _bits(kp_ref))
    assert torch.equal(_bits(vp_d.cpu()), _bits(vp_ref))
    # idempotent
    paged_ops.kv_append(k_new.to(gpu), v_new.to(gpu), kp_d, vp_d, slots.to(gpu))
    torch.cuda.synchronize()
    assert torch.equal(_bits(kp_d.cpu()), _bits(kp_ref))


def test_append_from_chunked_kv_view(gpu):
    """K and V as the two halves of one projection output
    (the reference's torch.chunk(key_value, 2, dim=-1)): strided rows."""
    n, gn, hd, nb, bs = 50, 8, 128, 10, 16
    g = torch.Generator().manual_seed(7)
    kv = torch.randn(n, 2 * gn * hd, generator=g).to(torch.bfloat16)
    k_new, v_new = (t.view(n, gn, hd) for t in torch.chunk(kv, 2, dim=-1))
    slots = torch.randperm(nb * bs, generator=g)[:n].to(torch.int64)
    slots[3] = -1          # padding row
    kp = torch.zeros(nb, gn, bs, hd, dtype=torch.bfloat16)
    vp = torch.zeros_like(kp)
    kp_ref, vp_ref = kp.clone(), vp.clone()
    oracle_paged.kv_append(kp_ref, vp_ref, k_new, v_new, slots)
    kv_d = kv.to(gpu)
    k_d, v_d = (t.view(n, gn, hd) for t in torch.chunk(kv_d, 2, dim=-1))
    kp_d, vp_d = kp.to(gpu), vp.to(gpu)
    paged_ops.kv_append(k_d, v_d, kp_d, vp_d, slots.to(gpu))
    torch.cuda.synchronize()
    assert torch.equal(kp_d.cpu().view(torch.int16), kp_ref.view(torch.int16))
    assert torch.equal(vp_d.cpu().view(torch.int16), vp_ref.view(torch.int16))


def test_append_token_major_pool(gpu):
    """The kernel follows the pool strides: a [nb, B, gn, hd] allocation viewed
    as [nb, gn, B, hd] works too."""
    n, gn, hd, nb, bs = 40, 4, 128, 6, 16
    k_new, v_new, slots = _case(n, gn, hd, nb, bs, torch.bfloat16, seed=3)
    kp = torch.zeros(nb, bs, gn, hd, dtype=torch.bfloat16).permute(0, 2, 1, 3)
    vp = torch.zeros(nb, bs, gn, hd, dtype=torch.bfloat16).permute(0, 2, 1, 3)
    kp_ref, vp_ref = kp.clone(), vp.clone()
    oracle_paged.kv_append(_bits(kp_ref), _bits(vp_ref), _bits(k_new), _bits(v_new), slots)
    kp_d = torch.zeros(nb, bs, gn, hd, dtype=torch.bfloat16, device=gpu).permute(0, 2, 1, 3)
    vp_d = torch.zeros(nb, bs, gn, hd, dtype=torch.bfloat16, device=gpu).permute(0, 2, 1, 3)
    paged_ops.kv_append(k_new.to(gpu), v_new.to(gpu), kp_d, vp_d, slots.to(gpu))
    torch.cuda.synchronize()
    assert torch.equal(_bits(kp_d.cpu().contiguous()), _bits(kp_ref.contiguous()))
    assert torch.equal(_bits(vp_d.cpu().contiguous()), _bits(vp_ref.contiguous()))
