"""Builds pathsig_amd/libpathsig_hip.so with hipcc (gfx950) and libpathsig_torch.so with g++, and installs the
Python package around them.

Counterpart of the reference's CMake build (`CMakeLists.txt`, `pyproject.toml`): `pip install .` or
`python setup.py build_py` compiles the HIP sources in-tree first; nothing is fetched.
"""
import importlib.util
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
        _build_library()
        super().run()


setup(
    name="pathsig-amd",
    version="0.1.0",
    description="Path signature and log-signature operators for AMD MI355X (gfx950), drop-in for pathsig",
    packages=["pathsig_amd"],
    package_data={"pathsig_amd": ["libpathsig_hip.so", "libpathsig_torch.so", "csrc/*.hip", "csrc/*.hpp", "csrc/*.cpp"]},
    data_files=[("include", ["include/pathsig_hip.h"])],
    python_requires=">=3.10",
    install_requires=["torch>=2.4"],
    cmdclass={"build_py": BuildWithHip},
)
