"""MI355X (gfx950) fused multi-head attention.

``capi``   ctypes binding of the C ABI (``libfmha_hip.so``)
``build``  in-tree build of the HIP library and the ``mha_manual`` torch extension
``load_ops()`` imports the extension so that ``torch.ops.mha_manual.*`` exists.
"""
import importlib.util
import os
import sys

__all__ = ["load_ops"]


def load_ops():
    """Import the in-tree ``mha_manual`` extension (registers torch.ops.mha_manual.*).

    Raises if it has not been built; there is no fallback implementation."""
    import torch
    if "mha_manual" in sys.modules:  # already imported (by this function or by `import mha_manual`)
        return torch.ops.mha_manual
    from . import build
    path = build.ext_path()
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: run `python -m nvfuserexamples_amd.build`")
    spec = importlib.util.spec_from_file_location("mha_manual", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    sys.modules["mha_manual"] = mod
    return torch.ops.mha_manual
