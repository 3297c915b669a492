"""Build recipe for the HIP library: hipcc, gfx950 only, in-tree output.

    python -m ironcore_amd.build

compiles every translation unit under ironcore_amd/csrc/ and links
ironcore_amd/lib/libironcore_paged.so.  Cross-compiles without a GPU.
"""
from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
LIB_DIR = PKG / "lib"
LIB_PATH = LIB_DIR / "libironcore_paged.so"
OBJ_DIR = PKG / "build" / "obj"

SOURCES = ["ic_api.hip", "kv_append.hip", "rope_kv_append.hip", "paged_decode.hip", "paged_decode_mfma.hip", "paged_prefill.hip",
           "paged_prefill_f32.hip", "mfma_probe.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-function",
    # the staging loads set m0 by hand and say so in their clobber lists
    "-Wno-inline-asm",
    # hipcc -O3 must not form packed-fp32 VALU ops on its own.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def csrc_digest() -> str:
    """SHA-256 over the names and contents of the kernel sources (csrc/*.hip,
    *.h): identifies the code a profiler figure was measured on."""
    import hashlib
    h = hashlib.sha256()
    for path in sorted(CSRC.glob("*")):
        if path.suffix in (".hip", ".h"):
            h.update(path.name.encode())
            h.update(b"\0")
            h.update(path.read_bytes())
            h.update(b"\0")
    return h.hexdigest()


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the HIP library cannot be built")
    return exe


# Per-file flags.  The prefill kernel keeps its MFMA accumulators in ordinary
# VGPRs: the softmax rescales them with VALU instructions, and the AGPR form
# costs a register copy each way per tile.
_VGPR_FORM = ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]
PER_SOURCE_FLAGS = {"paged_prefill.hip": _VGPR_FORM, "paged_prefill_f32.hip": _VGPR_FORM,
                    "paged_decode_mfma.hip": _VGPR_FORM}


def _compile(src: str, extra: list[str]) -> Path:
    obj = OBJ_DIR / (src + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, *PER_SOURCE_FLAGS.get(src, []), *extra, "-c", str(CSRC / src),
           "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{res.stdout}\n{res.stderr}")
    noise = "is not a recognized feature for this target"
    warn = "\n".join(line for line in res.stderr.splitlines() if noise not in line)
    if warn.strip():
        sys.stderr.write(warn + "\n")
    return obj


def build(verbose: bool = True, extra_flags: list[str] | None = None) -> Path:
    """Compile and link; returns the path of the shared library."""
    extra = list(extra_flags or [])
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    LIB_DIR.mkdir(parents=True, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objs = list(pool.map(lambda s: _compile(s, extra), SOURCES))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc",
           *map(str, objs), "-o", str(tmp)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} ({LIB_PATH.stat().st_size} bytes)")
    return LIB_PATH


if __name__ == "__main__":
    build()
