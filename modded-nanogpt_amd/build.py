"""Builds libngpt_fp8.so (all HIP kernels + the C ABI) for gfx950 with hipcc, in-tree.

    python -m modded_nanogpt_amd.build          # from the repository root

hipcc cross-compiles without a GPU.  The library lands in modded-nanogpt_amd/lib/ so it travels
with the source tree; nothing is installed into site-packages.
"""
from __future__ import annotations

import os
import pathlib
import shutil
import subprocess
import sys

PKG = pathlib.Path(__file__).resolve().parent
CSRC = PKG / "csrc"
LIB_DIR = PKG / "lib"
LIB_PATH = LIB_DIR / "libngpt_fp8.so"
BENCH_LIB_PATH = LIB_DIR / "libngpt_fp8_bench.so"     # + the timing aids behind NGPT_BENCH_BUILD, for measurements only
SOURCES = ["gemm_api.hip", "quant.hip", "ce.hip", "mlp_aux.hip", "bench_kernels.hip"]   # the last one is empty without NGPT_BENCH_BUILD

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # keep the compiler from forming packed-fp32 VALU ops out of scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and pathlib.Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or add /opt/rocm/bin to PATH)")


def build(verbose: bool = True, bench: bool = False) -> pathlib.Path:
    """Compile every HIP source into one shared library; always recompiles.  `bench`: the measurement build."""
    LIB_DIR.mkdir(exist_ok=True)
    srcs = [str(CSRC / s) for s in SOURCES if (CSRC / s).exists()]
    out = BENCH_LIB_PATH if bench else LIB_PATH
    tmp = out.with_suffix(".so.tmp")
    cmd = [hipcc_path(), *HIPCC_FLAGS, *(["-DNGPT_BENCH_BUILD"] if bench else []), "-I", str(PKG.parent / "include"),
           "-o", str(tmp), *srcs]
    if verbose:
        print("+", " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the device-only feature flag and says so once per file
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    os.replace(tmp, out)
    return out


if __name__ == "__main__":
    print(build())
    try:
        print(build(bench=True))
    except RuntimeError as e:      # only `bench.py --workload ceiling` needs it
        print("warning: the measurement build failed:", str(e)[:500], file=sys.stderr)
