"""Host-side checks that need no GPU: the C-ABI library loads and exports what
include/fmha_capi.h declares, argument validation returns the documented codes before
anything is launched, and the torch extension registers the reference's operator names
(reference fmha/fmha_manual.cpp:1240-1250)."""
import ctypes as C
import os
import re

import pytest
import torch

import oracle
from nvfuserexamples_amd import capi
from conftest import ROOT


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "fmha_capi.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fmha_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = capi.lib()
    names = _declared_functions()
    assert set(names) == set(capi.EXPORTS)
    for n in names:
        assert hasattr(L, n), n
    assert L.fmha_version().decode().count(".") == 1


def test_strerror_and_threshold():
    L = capi.lib()
    assert L.fmha_strerror(0) == b"ok"
    msgs = {L.fmha_strerror(c) for c in range(-8, 1)}
    assert len(msgs) == 9 and all(msgs)
    assert b"256" in L.fmha_strerror(-3) and b"unknown" in L.fmha_strerror(-99)
    for p in (0.0, 0.001, 0.05, 0.1, 0.25, 0.5, 0.9, 0.999):
        assert L.fmha_drop_threshold(p) == oracle.drop_threshold(p)
        assert L.fmha_drop_scale(p) == pytest.approx(oracle.drop_scale(p), rel=1e-7)
        assert L.fmha_drop_scale(p) * (256 - L.fmha_drop_threshold(p)) / 256 == pytest.approx(1.0, abs=1e-6)
    assert L.fmha_bwd_noalloc_max_rows() * 4 == 8 << 20


def test_workspace_query_without_a_gpu_says_no_pieces():
    """Where the device cannot be asked for its size (no GPU here) the forward never asks for a workspace,
    and nonsense parameter blocks get 0, not a crash."""
    L = capi.lib()
    P = capi.FwdParams()
    P.bh, P.sq, P.sk, P.d, P.scale = 4, 1, 8192, 64, 0.125
    if not torch.cuda.is_available():
        assert L.fmha_fwd_workspace_bytes(C.byref(P)) == 0
    P.d = 12
    assert L.fmha_fwd_workspace_bytes(C.byref(P)) == 0
    P.struct_bytes = 8
    assert L.fmha_fwd_workspace_bytes(C.byref(P)) == 0
    assert L.fmha_fwd_workspace_bytes(None) == 0


@pytest.mark.parametrize("bh,sq,sk,d,n,masked", [
    (4, 1, 4096, 64, 4, False), (3, 1, 1000, 128, 3, True), (2, 130, 520, 64, 2, True), (5, 3, 777, 96, 64, False),
    (1, 1, 131072, 128, 200, False), (7, 4, 300, 256, 2, True)])
def test_forced_pieces_size_their_workspace(bh, sq, sk, d, n, masked, monkeypatch):
    """FMHA_FWD_SPLIT=n needs no device: about n pieces (at most 64) of a multiple of 128 keys.  The workspace
    holds the partial outputs (fp32 for the decode kernel's shapes -- up to four query rows at head dim 64 /
    128 -- else the element type), their log-sum-exps and, for the matrix-pipe kernels only, a regrouped copy
    of a per-key mask; every part starts on a 256-byte boundary."""
    monkeypatch.setenv("FMHA_FWD_SPLIT", str(n))
    L = capi.lib()
    L.fmha_reload_overrides()
    try:
        P = capi.FwdParams()
        P.bh, P.sq, P.sk, P.d, P.scale = bh, sq, sk, d, 0.125
        if masked:
            P.mask_kind, P.mask_bh_div, P.mask_stride_b = capi.MASK_ADDITIVE, 1, sk
        got = L.fmha_fwd_workspace_bytes(C.byref(P))
        chunk = -(-(-(-sk // min(n, 64))) // 128) * 128
        pieces = -(-sk // chunk)
        decode = sq <= 4 and d in (64, 128)
        r256 = lambda x: (x + 255) // 256 * 256
        want = r256(bh * pieces * sq * d * (4 if decode else 2)) + r256(bh * pieces * sq * 4)
        if masked and not decode:
            want += r256(bh * pieces * chunk * 2)
        assert pieces >= 2 and got == want
        P.causal = 1
        assert L.fmha_fwd_workspace_bytes(C.byref(P)) == 0
    finally:
        monkeypatch.delenv("FMHA_FWD_SPLIT")
        L.fmha_reload_overrides()


def _valid_params():
    P = capi.FwdParams()
    P.q = P.k = P.v = P.o = 0x1000  # never dereferenced: every call below fails validation first
    P.bh, P.sq, P.sk, P.d = 2, 64, 64, 64
    P.dtype, P.scale = capi.F16, 0.125
    return P


@pytest.mark.parametrize("mutate,code", [
    (lambda P: setattr(P, "q", None), -1),
    (lambda P: setattr(P, "struct_bytes", 0), -5),                    # the struct must carry its size
    (lambda P: setattr(P, "struct_bytes", 64), -5),                   # ... at least up to the first release's fields
    (lambda P: setattr(P, "dtype", 7), -2),
    (lambda P: setattr(P, "d", 84), -3),                              # head dims: multiples of 8 ...
    (lambda P: setattr(P, "d", 264), -3),                             # ... up to 256
    (lambda P: setattr(P, "sq", 0), -3),
    (lambda P: setattr(P, "k", 0x1008), -4),
    (lambda P: setattr(P, "scale", 0.0), -5),
    (lambda P: setattr(P, "scale", float("nan")), -5),
    (lambda P: setattr(P, "mask_kind", 9), -5),
    (lambda P: setattr(P, "mask_kind", 1), -1),                       # mask kind without a pointer
    (lambda P: (setattr(P, "mask", 0x1000), setattr(P, "mask_kind", 2), setattr(P, "mask_bh_div", 1),
                setattr(P, "mask_neg", float("-inf"))), -5),         # 0/1 masks: mask_neg must be finite ...
    (lambda P: (setattr(P, "mask", 0x1000), setattr(P, "mask_kind", 2), setattr(P, "mask_bh_div", 1),
                setattr(P, "mask_neg", 5.0)), -5),                    # ... and not positive
    (lambda P: (setattr(P, "drop_kind", 1), setattr(P, "p_drop", 1.0)), -5),
    (lambda P: setattr(P, "drop_kind", 2), -1),                       # tensor dropout without a tensor
    (lambda P: (setattr(P, "save_softmax", 0x1000), setattr(P, "causal", 1)), -6),
    (lambda P: (setattr(P, "save_softmax", 0x1000), setattr(P, "drop_kind", 1), setattr(P, "p_drop", 0.1)), -6),
])
def test_forward_validation_codes(mutate, code):
    P = _valid_params()
    mutate(P)
    assert capi.lib().fmha_fwd_launch(C.byref(P), None) == code


def test_null_params_and_keep_mask_validation():
    L = capi.lib()
    assert L.fmha_fwd_launch(None, None) == -1
    assert L.fmha_bwd_launch(None, None) == -1
    assert L.fmha_philox_keep_mask(0, 0, 0.1, 1, 4, 4, None, None) == -1
    assert L.fmha_philox_keep_mask(0, 0, 1.5, 1, 4, 4, 0x1000, None) == -5
    assert L.fmha_philox_keep_mask(0, 0, 0.1, 0, 4, 4, 0x1000, None) == -3


def test_extension_registers_reference_operator_names():
    import mha_manual  # noqa: F401  (import registers the ops, as in reference test.py:2)
    for name in ("fmha_nvfuser", "fmha_train_nvfuser", "fmha_train_saveim_nvfuser", "fmha_fwd", "fmha_bwd",
                 "fmha_philox_keep_mask"):
        assert hasattr(torch.ops.mha_manual, name)
    s = torch.ops.mha_manual.fmha_train_saveim_nvfuser.default._schema
    assert [a.name for a in s.arguments] == ["input", "qk", "v", "pad_mask", "dropout_mask"]
    assert str(s.returns[0].type) == "List[Tensor]"
    s = torch.ops.mha_manual.fmha_nvfuser.default._schema
    assert [a.name for a in s.arguments] == ["input", "qk", "v", "amask"]


def test_cpu_tensors_are_rejected_loudly():
    """There is no CPU implementation behind the ops: CPU tensors must raise, not fall back."""
    import mha_manual  # noqa: F401
    z = torch.zeros(1, 4, 64, dtype=torch.float16)
    with pytest.raises((RuntimeError, NotImplementedError)):
        torch.ops.mha_manual.fmha_nvfuser(z, z, z, torch.zeros(1, 4, 4, dtype=torch.float16))


def test_package_has_no_oracle_dependency():
    """The shipped code may not import or call the CPU oracle."""
    pkg = os.path.join(ROOT, "nvfuserexamples_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".h", ".hip", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "import oracle" not in text and "from oracle" not in text and "fmha_oracle" not in text, f
    text = open(os.path.join(ROOT, "fmha", "fmha_manual.cpp")).read()
    assert "oracle" not in text
