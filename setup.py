"""Packaging entry point.  The reference builds `FGMS.backend` with torch's
CUDAExtension (setup.py:8-21: ext_modules + BuildExtension); here the same extension
module is declared to setuptools and built by fgms_amd.build, which drives hipcc for gfx950
directly (no source translation).  `pip install .`, `python setup.py install` and
`python setup.py build_ext [--inplace]` all produce FGMS/backend*.so and
fgms_amd/lib/libfgms_hip.so (the extension finds the library through a relative rpath)."""
import os
import shutil

from setuptools import Extension, setup
from setuptools.command.build_ext import build_ext

ROOT = os.path.dirname(os.path.abspath(__file__))


class BuildNative(build_ext):
    """Builds both shared objects in-tree (products newer than their sources are kept) and
    copies them to where the build or the install expects them."""

    def run(self):
        import sys
        sys.path.insert(0, ROOT)
        from fgms_amd import build
        build.build_all(verbose=True, force=False)
        if self.inplace:
            return
        for src in (build.torch_ext_path(), build.LIB_PATH):
            dst = os.path.join(self.build_lib, os.path.relpath(src, ROOT))
            os.makedirs(os.path.dirname(dst), exist_ok=True)
            shutil.copy2(src, dst)

    def get_outputs(self):
        import sys
        sys.path.insert(0, ROOT)
        from fgms_amd import build
        return [os.path.join(self.build_lib, os.path.relpath(p, ROOT)) for p in (build.torch_ext_path(), build.LIB_PATH)]


setup(
    name="FGMS",
    version="1.3+gfx950",
    packages=["FGMS", "fgms_amd"],
    # the sources are listed for sdists; BuildNative compiles them itself
    ext_modules=[Extension("FGMS.backend", sources=["fgms_amd/csrc/fgms_torch.cpp"])],
    cmdclass={"build_ext": BuildNative},
    zip_safe=False,
)
