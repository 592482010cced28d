"""Packaging entry point.  The reference builds `FGMS.backend` with torch's
CUDAExtension (setup.py:8-21); here the same module name is produced by
fgms_amd.build, which drives hipcc for gfx950 directly (no source translation)."""
from setuptools import Command, setup


class BuildNative(Command):
    description = "build libfgms_hip.so and FGMS.backend in-tree for gfx950"
    user_options = [("inplace", "i", "accepted for compatibility; the build is always in-tree")]

    def initialize_options(self):
        self.inplace = 1

    def finalize_options(self):
        pass

    def run(self):
        from fgms_amd import build
        build.build_all(verbose=True)


setup(
    name="FGMS",
    version="1.3+gfx950",
    packages=["FGMS", "fgms_amd"],
    package_data={"FGMS": ["*.so"], "fgms_amd": ["lib/*.so"]},
    cmdclass={"build_ext": BuildNative},
)
