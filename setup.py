"""Build script: compiles the hand-written HIP sources in dcnv4_amd/csrc into libdcnv4_gfx950.so with hipcc
for gfx950 and installs the pure-Python package around it.

Counterpart of the reference's DCNv4_op/setup.py:24-72, which drives torch's CUDAExtension; here there is no
torch extension machinery, no hipify pass and no CUDA path: `python setup.py build_ext` (or `develop` / `install`)
just runs dcnv4_amd/build.py.
"""
import importlib.util
import os

from setuptools import find_packages, setup
from setuptools.command.build_ext import build_ext as _build_ext

ROOT = os.path.dirname(os.path.abspath(__file__))


def _build_library(force=False):
    spec = importlib.util.spec_from_file_location("_dcnv4_amd_build", os.path.join(ROOT, "dcnv4_amd", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod.build(force=force)


class build_ext(_build_ext):
    def run(self):
        _build_library(force=bool(self.force))


setup(
    name="dcnv4_amd",
    version="0.1.0",
    description="DCNv4 and flash deformable attention operators for AMD MI355X (gfx950)",
    packages=find_packages(include=["dcnv4_amd", "dcnv4_amd.*", "DCNv4"]),
    package_data={"dcnv4_amd": ["libdcnv4_gfx950.so", "csrc/*", "functions/gfx950_table.json"]},
    cmdclass={"build_ext": build_ext},
    python_requires=">=3.8",
)
