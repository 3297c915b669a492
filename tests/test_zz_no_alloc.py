"""ic_paged_decode_static: the decode entry point that allocates nothing (its
split-K workspace is a static device array inside the library), called through
the C ABI and held to the output of ic_paged_decode on the same inputs and to
the oracle.  Collected last: it runs after every other GPU test has used the
library in this process, and it must also pass alone in a fresh process.

Bars: bit-identical to ic_paged_decode (same kernels, same grid: the wave cap
of the static variant is above what an MI355X launches), max-abs 2e-2 against
the oracle (bf16)."""
import math

import pytest
import torch

from ironcore_amd import _lib, workloads
from oracle import paged as oracle_paged

pytestmark = pytest.mark.gpu


def _abi_args(d, out):
    nb, gn, bs, hd = d.k_pool.shape
    sb, sh, st, _ = d.k_pool.stride()
    b, hn, _ = d.query.shape
    return [out.data_ptr(), out.stride(0), d.query.data_ptr(), d.query.stride(0),
            d.k_pool.data_ptr(), d.v_pool.data_ptr(), sb, sh, st,
            d.block_tables.data_ptr(), d.block_tables.stride(0), d.context_lens.data_ptr(),
            b, hn, gn, hd, bs, nb, d.max_context_len, 1.0 / math.sqrt(hd), 0]


def _both(wl, gpu):
    """(static entry point, existing entry point) on the same device tensors, raw C ABI."""
    lib = _lib.load()
    d = wl.to(gpu)
    b, hn, hd = d.query.shape
    stream = _lib.current_stream_ptr(gpu)
    dt = _lib.dtype_code(d.query.dtype)
    out_static = torch.full((b, hn * hd), float("nan"), dtype=d.query.dtype, device=gpu)
    out_plain = torch.full_like(out_static, float("nan"))
    need = lib.ic_paged_decode_workspace_bytes(b, hn, d.k_pool.shape[1], hd)
    ws = torch.empty(need, dtype=torch.uint8, device=gpu)
    torch.cuda.synchronize()
    rc = lib.ic_paged_decode_static(*_abi_args(d, out_static), dt, stream)
    assert rc == 0, lib.ic_error_string(rc)
    rc = lib.ic_paged_decode(*_abi_args(d, out_plain), ws.data_ptr(), ws.numel(), dt, stream)
    assert rc == 0, lib.ic_error_string(rc)
    torch.cuda.synchronize()
    return out_static.cpu(), out_plain.cpu()


def _hold(wl, out_static, out_plain):
    assert torch.isfinite(out_static.float()).all()
    assert torch.equal(out_static.view(torch.int16), out_plain.view(torch.int16)), \
        f"static vs ic_paged_decode: max|diff| {(out_static.float() - out_plain.float()).abs().max().item()}"
    ref = oracle_paged.paged_decode(wl.query, wl.k_pool, wl.v_pool, wl.block_tables, wl.context_lens)
    diff = (out_static.float() - ref.float()).abs().max().item()
    assert diff <= 2e-2, f"static vs oracle: max|diff| {diff}"


def test_static_decode_two_calls_second_smaller(gpu):
    """Two calls in a row on the one scratch array, the second with a smaller
    batch, fewer heads per group and shorter contexts: nothing the first call
    left in the array may show in the second."""
    big = workloads.make_decode_workload(24, 64, 8, 128, 900, 3000, seed=71)     # split rows: partials in use
    small = workloads.make_decode_workload(5, 8, 4, 128, 1, 400, seed=72)
    _hold(big, *_both(big, gpu))
    _hold(small, *_both(small, gpu))
    _hold(big, *_both(big, gpu))


def test_static_decode_mha_and_fp32(gpu):
    wl = workloads.make_decode_workload(9, 32, 32, 128, 500, 1500, seed=73)
    _hold(wl, *_both(wl, gpu))
    wl32 = workloads.make_decode_workload(4, 12, 12, 64, 30, 300, dtype=torch.float32, seed=74)
    lib = _lib.load()
    d = wl32.to(gpu)
    out = torch.empty(4, 12 * 64, dtype=torch.float32, device=gpu)
    rc = lib.ic_paged_decode_static(*_abi_args(d, out), _lib.dtype_code(torch.float32), _lib.current_stream_ptr(gpu))
    assert rc == 0, lib.ic_error_string(rc)
    torch.cuda.synchronize()
    ref = oracle_paged.paged_decode(wl32.query, wl32.k_pool, wl32.v_pool, wl32.block_tables, wl32.context_lens)
    assert (out.cpu() - ref).abs().max().item() <= 1e-4


def test_static_decode_rejects_oversized_batch(gpu):
    """Beyond the array: a clear error, nothing launched, the output untouched."""
    lib = _lib.load()
    wl = workloads.make_decode_workload(3, 64, 8, 128, 10, 40, seed=75)
    d = wl.to(gpu)
    out = torch.full((3, 64 * 128), 7.0, dtype=torch.bfloat16, device=gpu)
    args = _abi_args(d, out)
    args[12] = 4096                      # n_seqs the scratch cannot hold
    rc = lib.ic_paged_decode_static(*args, 0, _lib.current_stream_ptr(gpu))
    assert rc == -7 and b"static" in lib.ic_error_string(rc)
    torch.cuda.synchronize()
    assert (out == 7.0).all()
