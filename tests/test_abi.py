"""The C-ABI library: it loads without a GPU, exports every symbol the public
header declares, and rejects bad arguments on the host (no kernel is launched
by any call in this file)."""
import ctypes
import re
from pathlib import Path

import pytest

from ironcore_amd import _lib

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "ironcore_paged.h"


def _declared_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(ic_[a-z_0-9]+)\s*\(", text)))


def test_header_and_binding_agree():
    declared = _declared_functions()
    assert declared, "no declarations found in the header"
    assert declared == sorted(_lib.SIGNATURES)


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    for name in _declared_functions():
        assert hasattr(lib, name), f"{name} missing from {_lib.LIB_PATH}"


def test_version_and_error_strings():
    lib = _lib.load()
    assert lib.ic_version() >= 100
    assert lib.ic_error_string(0) == b"ok"
    for code in range(-7, 0):
        assert lib.ic_error_string(code) not in (b"", b"unknown error code")
    assert lib.ic_error_string(-99) == b"unknown error code"


def test_mfma_probe_rejects_bad_arguments():
    lib = _lib.load()
    assert lib.ic_mfma_probe(100, None, None) == -1      # no sink
    assert lib.ic_mfma_probe(0, 1 << 12, None) == -2     # no iterations
    assert lib.ic_mfma_probe(100, (1 << 12) + 2, None) == -6


def test_workspace_bytes():
    lib = _lib.load()
    assert lib.ic_paged_decode_workspace_bytes(0, 32, 32, 128) == 0
    assert lib.ic_paged_decode_workspace_bytes(64, 32, 5, 128) == 0          # hn % gn != 0
    small = lib.ic_paged_decode_workspace_bytes(1, 8, 8, 64)
    big = lib.ic_paged_decode_workspace_bytes(512, 28, 4, 128)
    assert 0 < small < big


DECODE_OK = dict(out=1 << 12, out_stride=4096, q=1 << 13, q_stride=4096, kp=1 << 14, vp=1 << 15,
                 sb=32 * 16 * 128, sh=16 * 128, st=128, bt=1 << 16, bt_stride=256, cl=1 << 17,
                 n=64, hn=32, gn=32, hd=128, bs=16, nb=1000, max_ctx=4096, scale=0.0884,
                 chunk=0, ws=1 << 20, ws_bytes=1 << 30, dtype=0)


def _decode(**over):
    a = dict(DECODE_OK, **over)
    return _lib.load().ic_paged_decode(
        a["out"], a["out_stride"], a["q"], a["q_stride"], a["kp"], a["vp"], a["sb"], a["sh"], a["st"],
        a["bt"], a["bt_stride"], a["cl"], a["n"], a["hn"], a["gn"], a["hd"], a["bs"], a["nb"],
        a["max_ctx"], a["scale"], a["chunk"], a["ws"], a["ws_bytes"], a["dtype"], None)


@pytest.mark.parametrize("over,code", [
    (dict(q=None), -1), (dict(bt=None), -1), (dict(out=None), -1),
    (dict(hn=30), -2), (dict(n=-1), -2), (dict(bt_stride=10), -2), (dict(out_stride=100), -2),
    (dict(chunk=24), -2), (dict(sb=0), -2),
    (dict(dtype=7), -3), (dict(hd=100), -3),
    (dict(ws=None), -4), (dict(ws_bytes=16), -4), (dict(ws=(1 << 20) + 64), -4),
    (dict(q=(1 << 13) + 2), -6), (dict(st=132, hd=128, dtype=2, sb=32 * 16 * 132 + 1), -6),
])
def test_decode_argument_errors(over, code):
    assert _decode(**over) == code


def test_decode_empty_batch_is_ok():
    assert _decode(n=0, q=None, out=None) == 0


def test_append_argument_errors():
    lib = _lib.load()

    def call(k_new=1 << 12, v_new=1 << 13, stride=4096, kp=1 << 14, vp=1 << 15, sb=65536, sh=2048,
             st=128, slots=1 << 16, n=8, gn=32, hd=128, bs=16, nb=100, dtype=0):
        return lib.ic_kv_append(k_new, v_new, stride, kp, vp, sb, sh, st, slots, n, gn, hd, bs, nb, dtype, None)
    assert call(n=0, k_new=None) == 0
    assert call(k_new=None) == -1
    assert call(slots=None) == -1
    assert call(n=-3) == -2
    assert call(stride=100) == -2
    assert call(dtype=9) == -3
    assert call(k_new=(1 << 12) + 4) == -6


def test_prefill_argument_errors():
    lib = _lib.load()

    def call(out=1 << 12, q=1 << 13, kp=1 << 14, vp=1 << 15, bt=1 << 16, cl=1 << 17, cu=1 << 18,
             n=4, chunk=512, hn=32, gn=32, hd=128, dtype=0, qs=4096, sb=65536, st=128, bs=16):
        return lib.ic_paged_prefill(out, 4096, q, qs, kp, vp, sb, 2048, st, bt, 300, cl, cu, n, chunk,
                                    hn, gn, hd, bs, 1000, 0.0884, 1, dtype, None)
    assert call(n=0, q=None) == 0
    assert call(cu=None) == -1
    assert call(hn=33) == -2
    assert call(qs=100) == -2
    assert call(dtype=5) == -3
    assert call(q=(1 << 13) + 8) == -6
    # the 16-bit kernel addresses inside a pool block with 32 bits: blocks of 4 GiB and more are refused
    assert call(sb=1 << 31) == -3
    assert call(st=1 << 24, bs=128) == -3


def test_masked_entry_points_argument_errors():
    """ic_paged_prefill_masked and ic_paged_decode_masked: a missing mask, negative
    strides, a mask row shorter than the keys it is said to cover, a key mask
    narrower than max_context_len and element types the kernels do not take are
    all refused on the host."""
    lib = _lib.load()

    def prefill(mask=1 << 19, s_seq=0, s_head=0, s_row=4608, keys=4608, dtype=0, n=4, q=1 << 13):
        return lib.ic_paged_prefill_masked(1 << 12, 4096, q, 4096, 1 << 14, 1 << 15, 65536, 2048, 128, 1 << 16, 300,
                                           1 << 17, 1 << 18, n, 512, 32, 32, 128, 16, 1000, 0.0884, mask, s_seq,
                                           s_head, s_row, keys, dtype, None)
    assert prefill(n=0, mask=None, q=None) == 0
    assert prefill(mask=None) == -1
    assert prefill(s_seq=-1) == -2
    assert prefill(s_head=-8) == -2
    assert prefill(s_row=-4608) == -2
    assert prefill(keys=-1) == -2
    assert prefill(s_row=100, keys=4608) == -2      # rows overlap the keys they are said to cover
    assert prefill(dtype=9) == -3

    def decode(key_mask=1 << 19, s_seq=4096, s_head=0, dtype=2, n=64, st=128, sb=32 * 16 * 128):
        a = DECODE_OK
        return lib.ic_paged_decode_masked(a["out"], a["out_stride"], a["q"], a["q_stride"], a["kp"], a["vp"], sb,
                                          a["sh"], st, a["bt"], a["bt_stride"], a["cl"], n, a["hn"], a["gn"],
                                          a["hd"], a["bs"], a["nb"], a["max_ctx"], a["scale"], 0, key_mask, s_seq,
                                          s_head, a["ws"], a["ws_bytes"], dtype, None)
    assert decode(n=0) == 0
    assert decode(key_mask=None) == -1
    assert decode(s_seq=4095) == -2                  # narrower than max_context_len
    assert decode(s_head=-1) == -2
    assert decode(dtype=0) == -3 and decode(dtype=1) == -3   # 16-bit calls use ic_paged_prefill_masked


def test_occupancy_query_counter_starts_at_zero_without_a_gpu():
    assert _lib.load().ic_decode_occupancy_queries() >= 0


def test_python_wrapper_rejects_cpu_tensors():
    import torch
    from ironcore_amd import paged_ops
    kp = torch.zeros(2, 1, 16, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU only"):
        paged_ops.paged_decode(torch.zeros(1, 1, 64, dtype=torch.bfloat16), kp, kp,
                               torch.zeros(1, 1, dtype=torch.int32), torch.ones(1, dtype=torch.int32), 1)
    with pytest.raises(RuntimeError, match="GPU only"):
        paged_ops.kv_append(torch.zeros(1, 1, 64, dtype=torch.bfloat16), torch.zeros(1, 1, 64, dtype=torch.bfloat16),
                            kp, kp, torch.zeros(1, dtype=torch.int64))


def _decode_static(**over):
    a = dict(DECODE_OK, **over)
    return _lib.load().ic_paged_decode_static(
        a["out"], a["out_stride"], a["q"], a["q_stride"], a["kp"], a["vp"], a["sb"], a["sh"], a["st"],
        a["bt"], a["bt_stride"], a["cl"], a["n"], a["hn"], a["gn"], a["hd"], a["bs"], a["nb"],
        a["max_ctx"], a["scale"], a["chunk"], a["dtype"], None)


def test_static_decode_scratch_limit():
    """The entry point on the library's own scratch refuses, on the host and
    before anything touches a GPU, a batch whose workspace exceeds the array."""
    lib = _lib.load()
    limit = 32 << 20
    # the BASELINE decode shapes fit
    for n, hn, gn in [(64, 32, 32), (128, 64, 8), (512, 28, 4)]:
        need = lib.ic_paged_decode_static_scratch_bytes(n, hn, gn, 128)
        assert 0 < need <= limit, (n, hn, gn, need)
        assert need <= lib.ic_paged_decode_workspace_bytes(n, hn, gn, 128)
    assert lib.ic_paged_decode_static_scratch_bytes(0, 32, 32, 128) == 0
    assert lib.ic_paged_decode_static_scratch_bytes(4096, 64, 8, 128) > limit
    assert _decode_static(n=4096, hn=64, gn=8, sb=8 * 16 * 128) == -7
    assert b"static" in lib.ic_error_string(-7)
    assert _decode_static(hn=30) == -2
    assert _decode_static(n=0, q=None, out=None) == 0
