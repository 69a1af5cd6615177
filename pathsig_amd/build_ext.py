"""Compiles pathsig_amd/csrc/*.hip for gfx950 into pathsig_amd/libpathsig_hip.so with hipcc.

Run `python -m pathsig_amd.build_ext` (or `__graft_entry__.build()`).  No torch headers are needed:
the library is a plain C-ABI shared object declared in include/pathsig_hip.h.
"""
from __future__ import annotations

import concurrent.futures
import pathlib
import subprocess
import sys

PKG = pathlib.Path(__file__).resolve().parent
CSRC = PKG / "csrc"
INCLUDE = PKG.parent / "include"
LIB = PKG / "libpathsig_hip.so"

SOURCES = ["api.hip", "words_kernels.hip", "batch_kernels.hip", "logsig_kernels.hip", "dense_kernels.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-munsafe-fp-atomics",
    # packed-fp32 VALU forms are kept out of every code object of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    f"-I{INCLUDE}",
    f"-I{CSRC}",
]


def _compile(src: str, verbose: bool) -> pathlib.Path:
    obj = CSRC / (src.rsplit(".", 1)[0] + ".o")
    cmd = ["hipcc", *HIPCC_FLAGS, "-c", str(CSRC / src), "-o", str(obj)]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
        raise RuntimeError(f"hipcc failed on {src}")
    if verbose and res.stderr.strip():
        lines = [ln for ln in res.stderr.splitlines() if "packed-fp32-ops" not in ln and ln.strip()]
        if lines:
            sys.stderr.write("\n".join(lines) + "\n")
    return obj


def build(verbose: bool = False, jobs: int = 4) -> pathlib.Path:
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile(s, verbose), SOURCES))
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *map(str, objs)]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
