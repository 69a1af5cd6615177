"""The built distribution carries the reference's import name: `python setup.py build_py` (with the in-tree
libraries reused) into a temporary directory, then `import pathsig` from there in a fresh interpreter
(`src/pathsig/__init__.py:5-8` is the surface to match)."""
from __future__ import annotations

import os
import pathlib
import subprocess
import sys

ROOT = pathlib.Path(__file__).resolve().parent.parent


def test_distribution_imports_as_pathsig(tmp_path):
    env = dict(os.environ, PATHSIG_SKIP_NATIVE_BUILD="1")
    build = subprocess.run([sys.executable, "setup.py", "-q", "build_py", "--build-lib", str(tmp_path / "lib"),
                            "egg_info", "--egg-base", str(tmp_path)], cwd=ROOT, env=env, capture_output=True, text=True,
                           timeout=600)
    assert build.returncode == 0, build.stderr
    pkg = tmp_path / "lib" / "pathsig"
    assert (pkg / "libpathsig_hip.so").is_file() and (pkg / "libpathsig_torch.so").is_file()
    code = (
        "import pathsig, torch\n"
        "assert pathsig.__all__ == ['Signature', 'LogSignature', 'projections']\n"
        "assert pathsig.__file__.startswith(%r)\n"
        "from pathsig import Signature, LogSignature, projections\n"
        "assert all(hasattr(projections, n) for n in ('words', 'anisotropic', 'lyndon'))\n"
        "for op in ('compute_signature', 'signature_backward', 'sig_to_logsig', 'logsig_backward'):\n"
        "    assert hasattr(torch.ops.pathsig, op)\n"
        "x = torch.empty(2, 5, 3, device='meta')\n"
        "e = torch.empty(0, dtype=torch.int64, device='meta')\n"
        "w = torch.empty(0, 2, dtype=torch.int32, device='meta')\n"
        "assert torch.ops.pathsig.compute_signature(x, 2, False, e, [], False, w).shape == (2, 12)\n"
        "print('ok')\n" % str(pkg))
    run = subprocess.run([sys.executable, "-c", code], cwd=tmp_path, env=dict(os.environ, PYTHONPATH=str(tmp_path / "lib")),
                         capture_output=True, text=True, timeout=600)
    assert run.returncode == 0 and run.stdout.strip() == "ok", run.stderr
