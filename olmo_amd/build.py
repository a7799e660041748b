"""Compiles the HIP sources under ``olmo_amd/csrc`` for gfx950 into ``olmo_amd/lib/libolmo355.so``.

Plain ``hipcc`` (no torch headers: the library's interface is the C-ABI of ``include/olmo355.h``).
Run ``python -m olmo_amd.build``; hipcc cross-compiles without a GPU.
"""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libolmo355.so")
SOURCES = ["w4_format.hip", "gemv.hip", "gemv_mid.hip", "relay.hip", "gemm.hip", "elementwise.hip", "attention.hip", "sample.hip", "beam.hip", "probe.hip"]

# -packed-fp32-ops off: keep the compiler from forming packed-fp32 VALU instructions
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.sep not in c or os.path.exists(c)):
            return c
    raise RuntimeError("hipcc not found")


def build(verbose: bool = True, jobs: int = 8) -> str:
    os.makedirs(LIBDIR, exist_ok=True)
    hipcc = _hipcc()
    objs = []

    def compile_one(src: str) -> str:
        obj = os.path.join(LIBDIR, src.replace(".hip", ".o"))
        cmd = [hipcc, *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
        if verbose and r.stderr.strip():
            # the host pass warns that it does not know the packed-fp32 target feature: harmless
            lines = [ln for ln in r.stderr.splitlines() if "packed-fp32-ops" not in ln and ln.strip()]
            if lines:
                print("\n".join(lines), file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=min(jobs, len(SOURCES))) as ex:
        objs = list(ex.map(compile_one, SOURCES))
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build()
