"""Builds libmoe_i8.so (HIP kernels + C-ABI) for gfx950 with hipcc, in-tree."""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "libmoe_i8.so"
SOURCES = ["align.hip", "quant.hip", "sum.hip", "router.hip", "gemm_stream.hip", "gemm_tile.hip", "gemm_narrow.hip", "api.hip"]
PROBE_LIB_PATH = PKG_DIR / "libmoe_i8_probe.so"  # the benchmark's MFMA rate probe, a library of its own

# packed-fp32 VALU ops are switched off for all device code (hipcc's host pass warns that it does
# not know the feature; that is harmless).
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-inline-asm",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + proc.stdout + proc.stderr)


def build_library(verbose: bool = False) -> Path:
    """Compile every source to an object file and link the shared library. Always rebuilds."""
    hipcc = _hipcc()
    objdir = PKG_DIR / "build"
    objdir.mkdir(exist_ok=True)
    objs = [objdir / (Path(s).stem + ".o") for s in SOURCES]
    probe_obj = objdir / "probe.o"

    def compile_one(pair):
        src, obj = pair
        cmd = [hipcc, *HIPCC_FLAGS, "-c", str(CSRC / src), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd), flush=True)
        _run(cmd)

    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES) + 1)) as pool:
        list(pool.map(compile_one, zip([*SOURCES, "probe.hip"], [*objs, probe_obj])))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objs), "-o", str(tmp)])
    os.replace(tmp, LIB_PATH)
    tmp = PROBE_LIB_PATH.with_suffix(".so.tmp")
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", str(probe_obj), "-o", str(tmp)])
    os.replace(tmp, PROBE_LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose="-v" in sys.argv))
