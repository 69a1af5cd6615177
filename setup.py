"""Builds pathsig_amd/libpathsig_hip.so with hipcc (gfx950) and libpathsig_torch.so with g++, and installs the
Python package around them.

Counterpart of the reference's CMake build (`CMakeLists.txt`, `pyproject.toml`): `pip install .` or
`python setup.py build_py` compiles the HIP sources in-tree first; nothing is fetched.

The distribution installs the package under the reference's import name, `pathsig` (the source directory is
`pathsig_amd/`), so `import pathsig` and `from pathsig import Signature, LogSignature, projections` work
unchanged.  `PATHSIG_SKIP_NATIVE_BUILD=1` reuses the libraries already built in-tree instead of compiling.
"""
import importlib.util
import os
import pathlib

from setuptools import setup
from setuptools.command.build_py import build_py

ROOT = pathlib.Path(__file__).resolve().parent


def _build_library():
    spec = importlib.util.spec_from_file_location("_pathsig_build_ext", ROOT / "pathsig_amd" / "build_ext.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    mod.build(verbose=True)
    return mod.build_torch_ops(verbose=True)


class BuildWithHip(build_py):
    def run(self):
        if not os.environ.get("PATHSIG_SKIP_NATIVE_BUILD"):
            _build_library()
        for lib in ("libpathsig_hip.so", "libpathsig_torch.so"):
            if not (ROOT / "pathsig_amd" / lib).is_file():
                raise RuntimeError(f"pathsig_amd/{lib} is not built")
        super().run()


setup(
    name="pathsig-amd",
    version="0.1.0",
    description="Path signature and log-signature operators for AMD MI355X (gfx950), drop-in for pathsig",
    packages=["pathsig"],
    package_dir={"pathsig": "pathsig_amd"},
    package_data={"pathsig": ["libpathsig_hip.so", "libpathsig_torch.so", "csrc/*.hip", "csrc/*.hpp", "csrc/*.cpp"]},
    data_files=[("include", ["include/pathsig_hip.h"])],
    python_requires=">=3.10",
    install_requires=["torch>=2.4"],
    cmdclass={"build_py": BuildWithHip},
)
