"""`python setup.py build` (what `install` copies from; reference README.md:5-7, setup.py:7-18) yields an
importable `mha_manual` together with the library it links: checked in a fresh interpreter whose only
path entry is the build directory.  The objects of the in-tree build are reused (FMHA_BUILD_ONLY matches
no object) so that the test exercises the packaging, not the compiler, and stays short."""
import glob
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_setup_build_produces_an_importable_module(tmp_path):
    env = dict(os.environ, FMHA_BUILD_ONLY="no-object-has-this-name")
    base = str(tmp_path / "b")
    r = subprocess.run([sys.executable, "setup.py", "-q", "build", "--build-base", base], cwd=ROOT, env=env,
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=1500)
    assert r.returncode == 0, r.stdout[-3000:]
    libdirs = glob.glob(os.path.join(base, "lib*"))
    assert len(libdirs) == 1, libdirs
    lib = libdirs[0]
    assert glob.glob(os.path.join(lib, "mha_manual*.so"))
    assert os.path.exists(os.path.join(lib, "nvfuserexamples_amd", "lib", "libfmha_hip.so"))
    assert os.path.exists(os.path.join(lib, "nvfuserexamples_amd", "capi.py"))
    code = ("import sys; sys.path[:] = [p for p in sys.path if 'repo' not in p]; sys.path.insert(0, %r); "
            "import torch, mha_manual; assert %r in mha_manual.__file__; "
            "ops = torch.ops.mha_manual; "
            "[getattr(ops, n) for n in ('fmha_nvfuser', 'fmha_train_nvfuser', 'fmha_train_saveim_nvfuser', 'fmha_fwd', 'fmha_bwd')]; "
            "from nvfuserexamples_amd import capi; assert %r in capi.LIB_PATH; capi.lib().fmha_version()" % (lib, lib, lib))
    r = subprocess.run([sys.executable, "-c", code], cwd=str(tmp_path), stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                       text=True, timeout=600, env={k: v for k, v in os.environ.items() if k != "PYTHONPATH"})
    assert r.returncode == 0, r.stdout[-3000:]
