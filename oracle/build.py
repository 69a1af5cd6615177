"""Compile oracle/ref_words.c (fp64 and fp32 variants) into oracle/liboracle_words.so with gcc.

Test infrastructure only.  Run as `python -m oracle.build` or through `__graft_entry__.build()`.
"""
from __future__ import annotations

import pathlib
import subprocess

HERE = pathlib.Path(__file__).resolve().parent
LIB = HERE / "liboracle_words.so"


def build(verbose: bool = False) -> pathlib.Path:
    src = HERE / "ref_words.c"
    objs = []
    for real, suf in (("double", "_f64"), ("float", "_f32")):
        obj = HERE / f"ref_words{suf}.o"
        cmd = ["gcc", "-O2", "-fPIC", "-fopenmp", "-std=c11", "-ffp-contract=off",
               f"-DREAL={real}", f"-DSUF={suf}", "-c", str(src), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd))
        subprocess.run(cmd, check=True)
        objs.append(str(obj))
    cmd = ["gcc", "-shared", "-fopenmp", "-o", str(LIB), *objs]
    if verbose:
        print(" ".join(cmd))
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
