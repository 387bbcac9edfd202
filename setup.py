"""Install-time build of genbmm_amd: compiles the HIP sources for gfx950 with hipcc
(genbmm_amd/build.py) and ships the shared library inside the package.

    python setup.py build        # or: pip install --no-build-isolation .

Takes the place of the reference's setup.py (a torch CUDAExtension named `_genbmm`,
setup.py:1-27); there is no Python extension module here, only libgenbmm_gfx950.so,
which genbmm_amd/_lib.py loads with ctypes.  The C header is installed next to it.
"""
import os
import shutil

from setuptools import setup
from setuptools.command.build_py import build_py as _build_py

ROOT = os.path.dirname(os.path.abspath(__file__))


class build_py(_build_py):
    def run(self):
        import importlib.util

        spec = importlib.util.spec_from_file_location("genbmm_amd_build", os.path.join(ROOT, "genbmm_amd", "build.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)   # torch is not needed to compile
        mod.build(verbose=False)
        inc = os.path.join(ROOT, "genbmm_amd", "include")
        os.makedirs(inc, exist_ok=True)
        shutil.copy(os.path.join(ROOT, "include", "genbmm_gfx950.h"), inc)
        super().run()


setup(
    name="genbmm_amd",
    version="0.1",
    description="Generalized-semiring batched matmul for MI355X (gfx950): drop-in for harvardnlp/genbmm",
    packages=["genbmm_amd"],
    package_data={"genbmm_amd": ["lib/*.so", "include/*.h"]},
    cmdclass={"build_py": build_py},
    python_requires=">=3.9",
)
