"""Install recipe: ``pip install --no-build-isolation .`` builds the HIP library and the
``flash_gaussian_splatting`` extension for gfx950 with hipcc / g++ (``flashgs_amd/build.py``; no
CUDAExtension, no hipify) and installs them with the ``flashgs_amd`` package, the way FlashGS's own
``setup.py:32-48`` installs its extension.  The extension finds ``libflashgs_hip.so`` through its
``$ORIGIN/flashgs_amd/lib`` run path, so the two land side by side in site-packages.

``FLASHGS_AMD_REUSE_BUILT=1`` installs the binaries already built in the tree instead of compiling.
"""
import os
import shutil
import sys

from setuptools import Extension, setup
from setuptools.command.build_ext import build_ext
from setuptools.command.build_py import build_py

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

_built = False


def native_build():
    global _built
    if _built:
        return
    from flashgs_amd import build as b
    reuse = os.environ.get("FLASHGS_AMD_REUSE_BUILT") == "1"
    if not (reuse and os.path.exists(b.LIB_PATH) and os.path.exists(b.ext_path())):
        b.build_all()
    _built = True


class BuildPy(build_py):
    """The package data (the shared libraries) has to exist before it is collected."""

    def run(self):
        native_build()
        super().run()


class BuildExt(build_ext):
    def build_extension(self, ext):
        native_build()
        from flashgs_amd import build as b
        dst = self.get_ext_fullpath(ext.name)
        os.makedirs(os.path.dirname(dst), exist_ok=True)
        shutil.copy2(b.ext_path(), dst)


setup(
    name="flash_gaussian_splatting",
    version="0.2.0",
    description="MI355X (gfx950) forward rasterizer behind FlashGS's flash_gaussian_splatting op surface",
    packages=["flashgs_amd"],
    package_data={"flashgs_amd": ["lib/*.so", "csrc/*"]},
    ext_modules=[Extension("flash_gaussian_splatting", sources=[])],
    cmdclass={"build_py": BuildPy, "build_ext": BuildExt},
    python_requires=">=3.8",
    zip_safe=False,
)
