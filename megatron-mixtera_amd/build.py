"""Build recipe for the C-ABI library: every ``csrc/*.hip`` file -> one shared object.

``hipcc`` cross-compiles for gfx950 without a GPU, so this runs anywhere the ROCm
toolchain is installed.  The result, ``libmi355_decode.so``, sits next to this file and
is what :mod:`_lib` loads.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
INCLUDE = PKG_DIR.parent / "include"   # the public header: every entry point is compiled against it
LIB_NAME = "libmi355_decode.so"
LIB_PATH = PKG_DIR / LIB_NAME
# measurement aids of bench.py (a streaming-read kernel); not part of the product library or its ABI
BENCH_LIB_PATH = PKG_DIR / "libmi355_bench.so"

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # packed fp32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found: the HIP kernels cannot be built")


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _run(cmd: list[str], verbose: bool) -> None:
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    noise = ("packed-fp32-ops", "'-packed-fp32-ops' is not a recognized feature")
    out = "\n".join(l for l in proc.stdout.splitlines() if not any(n in l for n in noise))
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{out}")
    if verbose and out.strip():
        print(out)


def _hipcc(inputs: list[Path], output: Path, verbose: bool) -> None:
    """Compile every source to an object (in parallel: one hipcc per file), then link the shared object."""
    flags = [f for f in HIPCC_FLAGS if f != "-shared"]
    with tempfile.TemporaryDirectory(prefix="mi355_build_") as tmp:
        objects = [Path(tmp) / (src.stem + ".o") for src in inputs]
        jobs = [[hipcc_path(), *flags, "-I", str(CSRC), "-I", str(INCLUDE), "-c", str(src), "-o", str(obj)]
                for src, obj in zip(inputs, objects)]
        with ThreadPoolExecutor(max_workers=min(len(jobs), os.cpu_count() or 1, 16)) as pool:
            list(pool.map(lambda cmd: _run(cmd, verbose), jobs))
        _run([hipcc_path(), "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objects), "-o", str(output)], verbose)


def build_library(verbose: bool = False) -> Path:
    """Compile all kernels into ``libmi355_decode.so`` and the benchmark's measurement kernels into
    ``libmi355_bench.so`` (always recompiles)."""
    _hipcc(sources(), LIB_PATH, verbose)
    _hipcc(sorted((CSRC / "bench").glob("*.hip")), BENCH_LIB_PATH, verbose)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose="-v" in sys.argv))
