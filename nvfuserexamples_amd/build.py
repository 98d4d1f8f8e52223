"""In-tree build of the native parts.

``build_hip()``  hipcc -> ``nvfuserexamples_amd/lib/libfmha_hip.so`` (HIP kernels + C ABI)
``build_ext()``  g++   -> ``mha_manual.<abi>.so`` at the repository root: the host-only
                 torch extension that registers ``torch.ops.mha_manual.*`` and calls the
                 C ABI (same module name and source path as the reference's setup.py:7-18)

Everything is compiled for gfx950 only.  Run as ``python -m nvfuserexamples_amd.build``.
"""
import concurrent.futures as cf
import os
import re
import subprocess
import sys
import sysconfig

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
LIBDIR = os.path.join(PKG, "lib")
OBJDIR = os.path.join(ROOT, "build", "obj")
HIP_LIB = os.path.join(LIBDIR, "libfmha_hip.so")
EXTRA = os.environ.get("FMHA_EXTRA_HIPFLAGS", "").split()  # experiments only

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed fp32 VALU forms stay off on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # keep MFMA accumulators in architectural VGPRs (no AGPR round trips before the softmax VALU work)
    "-mllvm", "-amdgpu-mfma-vgpr-form",
    # the kernels use +-inf deliberately but never produce or consume NaN
    "-fno-honor-nans",
    "-Wno-unused-command-line-argument",
]


def _tus():
    """(source, object name, extra defines) for every translation unit of the library."""
    tus = [("fmha_capi.hip", "fmha_capi.o", []), ("fmha_fwd_fp8.hip", "fmha_fwd_fp8.o", []),
           ("fmha_fwd_decode.hip", "fmha_fwd_decode.o", []), ("fmha_probe.hip", "fmha_probe.o", [])]
    for bf in (0, 1):
        for d in (64, 128, 256):
            for strided in (0, 1):  # folded contiguous tensors / row layouts given at run time
                tag = f"{'bf16' if bf else 'f16'}_d{d}" + ("_strided" if strided else "")
                defs = [f"-DFMHA_TU_BF16={bf}", f"-DFMHA_TU_D={d}", f"-DFMHA_TU_STRIDED={strided}"]
                tus.append(("fmha_fwd.hip", f"fmha_fwd_{tag}.o", defs))
                tus.append(("fmha_bwd.hip", f"fmha_bwd_{tag}.o", defs))
    return tus


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(ln for ln in r.stdout.splitlines() if "packed-fp32-ops" not in ln)
    if r.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + out)
    return out


def build_hip(jobs=None, verbose=True):
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    cmds, objs = [], []
    only = os.environ.get("FMHA_BUILD_ONLY")  # development aid: regex of objects to recompile
    for src, obj, defs in _tus():
        o = os.path.join(OBJDIR, obj)
        objs.append(o)
        if only and os.path.exists(o) and not re.search(only, obj):
            continue
        cmds.append([HIPCC, *HIP_FLAGS, *EXTRA, *defs, "-c", os.path.join(CSRC, src), "-o", o])
    with cf.ThreadPoolExecutor(jobs) as ex:
        for out in ex.map(_run, cmds):
            if verbose and out.strip():
                print(out)
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", HIP_LIB, *objs])
    if verbose:
        print("built", HIP_LIB)
    return HIP_LIB


def ext_path():
    suffix = sysconfig.get_config_var("EXT_SUFFIX")
    return os.path.join(ROOT, "mha_manual" + suffix)


def build_ext(verbose=True):
    """Host-only torch extension; links libfmha_hip.so through an $ORIGIN rpath."""
    from torch.utils import cpp_extension as ce
    import torch

    src = os.path.join(ROOT, "fmha", "fmha_manual.cpp")
    out = ext_path()
    inc = []
    for p in ce.include_paths() + [sysconfig.get_paths()["include"], ROOT, "/opt/rocm/include"]:
        inc += ["-I", p]
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = [
        "g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=mha_manual",
        "-DTORCH_API_INCLUDE_EXTENSION_H", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
        *inc, src, "-o", out,
        "-L", LIBDIR, "-lfmha_hip", "-L", torch_lib, "-L", "/opt/rocm/lib",
        "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python", "-lamdhip64",
        "-Wl,-rpath,$ORIGIN/nvfuserexamples_amd/lib", f"-Wl,-rpath,{torch_lib}", "-Wl,-rpath,/opt/rocm/lib",
    ]
    _run(cmd)
    if verbose:
        print("built", out)
    return out


def build_all(verbose=True):
    build_hip(verbose=verbose)
    build_ext(verbose=verbose)


if __name__ == "__main__":
    if len(sys.argv) > 1 and sys.argv[1] == "hip":
        build_hip()
    elif len(sys.argv) > 1 and sys.argv[1] == "ext":
        build_ext()
    else:
        build_all()
