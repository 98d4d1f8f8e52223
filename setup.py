"""Builds and installs the `mha_manual` extension module, as the reference's setup.py does
(reference setup.py:7-18, README.md:5-7: `python setup.py install`, then `import mha_manual`), but
for ROCm: the HIP kernels and their C ABI go into libfmha_hip.so (hipcc, gfx950) and the host-only
operator registration in fmha/fmha_manual.cpp is compiled with the C++ compiler and linked to it.

    python setup.py install                  # module mha_manual + package nvfuserexamples_amd (with lib/libfmha_hip.so)
    python setup.py build                    # the same files under build/lib*
    python setup.py build_ext --inplace      # in-tree build (what the tests load)

mha_manual.*.so finds the library through the rpath $ORIGIN/nvfuserexamples_amd/lib, which holds in the
source tree, under build/lib* and in site-packages alike.
"""
import os
import shutil

from setuptools import Extension, setup
from setuptools.command.build_ext import build_ext as _build_ext


class BuildNative(_build_ext):
    """Runs the project's own build (hipcc / g++) and puts its products where setuptools expects them."""

    def run(self):
        from nvfuserexamples_amd import build
        build.build_all()
        dst = self.get_ext_fullpath("mha_manual")
        if os.path.abspath(dst) != os.path.abspath(build.ext_path()):
            os.makedirs(os.path.dirname(dst), exist_ok=True)
            shutil.copy2(build.ext_path(), dst)
        if not self.inplace:
            libdir = os.path.join(self.build_lib, "nvfuserexamples_amd", "lib")
            os.makedirs(libdir, exist_ok=True)
            shutil.copy2(build.HIP_LIB, libdir)

    def get_outputs(self):
        out = [self.get_ext_fullpath("mha_manual")]
        if not self.inplace:
            out.append(os.path.join(self.build_lib, "nvfuserexamples_amd", "lib", "libfmha_hip.so"))
        return out


setup(
    name="mha_manual",
    version="0.2",
    description="gfx950 fused multi-head attention behind torch.ops.mha_manual",
    packages=["nvfuserexamples_amd"],
    # no sources: BuildNative compiles fmha/fmha_manual.cpp and the HIP translation units itself
    ext_modules=[Extension("mha_manual", sources=[])],
    cmdclass={"build_ext": BuildNative},
    zip_safe=False,
)
