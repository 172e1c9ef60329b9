"""Ahead-of-time build of the HIP engine for gfx950 (replaces the reference's
per-config JIT build, xlstm/blocks/slstm/src/cuda_init.py:60-117).

``python -m xlstm_amd.build`` compiles ``csrc/*.hip`` with hipcc into
``xlstm_amd/lib/libxlstm_amd.so``.  hipcc cross-compiles, so no GPU is needed.
"""
from __future__ import annotations

import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
SOURCES = [os.path.join(PKG, "csrc", "slstm_hip.hip")]
LIB = os.path.join(PKG, "lib", "libxlstm_amd.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-shared", "-fPIC",
    # the compiler must not form packed-fp32 instructions from scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    # the LDS-direct loads are inline assembly that sets M0 and says so in its clobber list
    "-Wno-inline-asm",
]


def build(verbose: bool = False, extra_flags=(), out: str = LIB) -> str:
    """Builds the engine and returns the path of the library.  ``extra_flags`` / ``out`` are for the two measurement
    builds the kernels know about: ``-DXS_PROFILE`` (per-phase cycle stamps, read back by ``bench.py --phase-profile``) and
    ``-DXS_SMALL_BATCH_FMA`` (the FMA contraction for row tiles of 4 rows); from the command line:
    ``python -m xlstm_amd.build -DXS_PROFILE -o xlstm_amd/lib/libxlstm_amd_profile.so``."""
    hipcc = os.environ.get("HIPCC", "hipcc")
    os.makedirs(os.path.dirname(out), exist_ok=True)
    cmd = [hipcc, *HIPCC_FLAGS, *extra_flags, "-I", os.path.join(ROOT, "include"), "-o", out, *SOURCES]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    log = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{log}")
    if verbose and log.strip():
        print(log)
    return out


if __name__ == "__main__":
    argv = sys.argv[1:]
    target = LIB
    if "-o" in argv:
        i = argv.index("-o")
        target = os.path.abspath(argv[i + 1])
        del argv[i:i + 2]
    print(build(verbose=True, extra_flags=tuple(argv), out=target))
    sys.exit(0)
