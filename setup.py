"""Builds the `mha_manual` extension module, as the reference's setup.py does, but for ROCm:
the HIP kernels and their C ABI go into libfmha_hip.so (hipcc, gfx950) and the host-only
operator registration in fmha/fmha_manual.cpp is compiled with the C++ compiler and linked to it.

    python setup.py build_ext --inplace      # in-tree build (what the tests load)
"""
from setuptools import Command, setup


class BuildNative(Command):
    description = "build libfmha_hip.so and the mha_manual extension in-tree"
    user_options = [("inplace", "i", "accepted for compatibility; the build is always in-tree")]

    def initialize_options(self):
        self.inplace = True

    def finalize_options(self):
        pass

    def run(self):
        from nvfuserexamples_amd import build
        build.build_all()


setup(
    name="mha_manual",
    version="0.1",
    description="gfx950 fused multi-head attention behind torch.ops.mha_manual",
    packages=["nvfuserexamples_amd"],
    cmdclass={"build_ext": BuildNative},
)
