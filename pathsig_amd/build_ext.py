"""Compiles pathsig_amd/csrc/*.hip for gfx950 into pathsig_amd/libpathsig_hip.so with hipcc, and the torch
operator registration csrc/torch_ops.cpp into pathsig_amd/libpathsig_torch.so with g++.

Run `python pathsig_amd/build_ext.py` (or `__graft_entry__.build()`).  The first library needs no torch headers:
it is a plain C-ABI shared object declared in include/pathsig_hip.h.  The second one links against it and against
the torch libraries of the running interpreter.
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
TORCH_LIB = PKG / "libpathsig_torch.so"

# (source, object, extra flags).  dense_kernels.hip is compiled once per group of register-tiled shapes and once
# for the table of shapes and the dispatch, so the shapes build in parallel (the largest objects come first).
DENSE_GROUPS = 8  # kDenseGroups of csrc/dense.hpp
UNITS = ([("dense_kernels.hip", f"dense_kernels_g{g}.o", [f"-DPSIG_GROUP={g}"]) for g in range(DENSE_GROUPS)]
         + [("batch_kernels.hip", "batch_kernels.o", []), ("words_kernels.hip", "words_kernels.o", []),
            ("logsig_kernels.hip", "logsig_kernels.o", []), ("dense_kernels.hip", "dense_kernels.o", []),
            ("api.hip", "api.o", [])])

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


def _compile(unit, verbose: bool, obj_dir: pathlib.Path, defines) -> pathlib.Path:
    src, obj_name, extra = unit
    obj = obj_dir / obj_name
    cmd = ["hipcc", *HIPCC_FLAGS, *defines, *extra, "-c", str(CSRC / src), "-o", str(obj)]
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


def build(verbose: bool = False, jobs: int = 8, only=None, out_dir: pathlib.Path | None = None) -> pathlib.Path:
    """only: iterable of (d, depth) pairs; the register-tiled kernels are then compiled for these shapes alone (a
    small library that builds in a minute; every other shape runs on the per-word kernels).
    out_dir: where the objects and the library go (default: beside the sources / in the package)."""
    defines = []
    if only:
        defines = ["-DPSIG_ONLY=" + ",".join("{%d,%d}" % (int(d), int(n)) for d, n in only)]
    lib = LIB if out_dir is None else pathlib.Path(out_dir) / LIB.name
    obj_dir = CSRC if out_dir is None else pathlib.Path(out_dir) / "obj"
    obj_dir.mkdir(parents=True, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda u: _compile(u, verbose, obj_dir, defines), UNITS))
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(lib), *map(str, objs)]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return lib


def build_torch_ops(verbose: bool = False, out_dir: pathlib.Path | None = None) -> pathlib.Path:
    """C++ registration of the operators with the torch dispatcher (host code only; needs libpathsig_hip.so)."""
    import torch
    from torch.utils import cpp_extension

    if torch.version.hip is None:
        raise RuntimeError("the operator library needs a ROCm build of PyTorch")
    includes = [f"-I{p}" for p in cpp_extension.include_paths()] + ["-I/opt/rocm/include", f"-I{INCLUDE}"]
    lib_dirs = cpp_extension.library_paths()
    pkg = PKG if out_dir is None else pathlib.Path(out_dir)
    torch_lib = pkg / TORCH_LIB.name
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}", *includes,
           str(CSRC / "torch_ops.cpp"), "-o", str(torch_lib),
           *[f"-L{d}" for d in lib_dirs], "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch",
           f"-L{pkg}", "-lpathsig_hip", "-Wl,-rpath,$ORIGIN", *[f"-Wl,-rpath,{d}" for d in lib_dirs]]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
        raise RuntimeError("g++ failed on torch_ops.cpp")
    return torch_lib


if __name__ == "__main__":
    import argparse

    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--only", default=None, metavar="DxN[,DxN...]",
                    help="compile the register-tiled kernels for these (d, depth) shapes only, e.g. 4x6,8x4")
    ap.add_argument("--out-dir", default=None, help="directory for the objects and the two libraries")
    opts = ap.parse_args()
    shapes = [tuple(int(v) for v in item.split("x")) for item in opts.only.split(",")] if opts.only else None
    print(build(verbose=True, only=shapes, out_dir=opts.out_dir))
    print(build_torch_ops(verbose=True, out_dir=opts.out_dir))
