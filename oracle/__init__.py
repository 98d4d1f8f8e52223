"""ctypes front end of the CPU oracle (``oracle/fmha_oracle.c``).

TEST INFRASTRUCTURE ONLY.  Importers are restricted to ``tests/``, the smoke
check and the benchmark's CPU-baseline leg; the shipped package never imports
this module and has no CPU fallback.

The functions mirror the reference's ground-truth compositions
(reference test.py:12-18 and test_train_mha.py:14-21) generalised over shape,
mask layout, causal masking and seeded dropout, with double accumulation.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libfmha_oracle.so")


def build(force=False):
    """Compile the C restatement with gcc (a few hundred ms)."""
    src = os.path.join(_HERE, "fmha_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-s", "-B"])
    return _LIB_PATH


class _Params(C.Structure):
    _fields_ = [
        ("bh", C.c_int64), ("sq", C.c_int64), ("sk", C.c_int64), ("d", C.c_int64),
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p),
        ("mask", C.c_void_p),
        ("mask_bh_div", C.c_int64), ("mask_sb", C.c_int64), ("mask_sq", C.c_int64),
        ("mask_kind", C.c_int32), ("mask_neg", C.c_float),
        ("causal", C.c_int32), ("scale", C.c_float),
        ("drop_kind", C.c_int32), ("drop_mask", C.c_void_p),
        ("p_drop", C.c_float), ("drop_scale", C.c_float),
        ("seed", C.c_uint64), ("offset", C.c_uint64),
        ("round_p", C.c_int32), ("round_o", C.c_int32),
        ("o", C.c_void_p), ("lse", C.c_void_p), ("softmax", C.c_void_p), ("dropout", C.c_void_p),
        ("dout", C.c_void_p), ("dq", C.c_void_p), ("dk", C.c_void_p), ("dv", C.c_void_p),
        ("bh_offset", C.c_int64),
    ]


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.fmha_oracle_fwd.argtypes = [C.POINTER(_Params)]
        _lib.fmha_oracle_bwd.argtypes = [C.POINTER(_Params)]
        _lib.fmha_oracle_philox4x32_10.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        _lib.fmha_oracle_keep_mask.argtypes = [C.c_uint64, C.c_uint64, C.c_float, C.c_int64,
                                               C.c_int64, C.c_int64, C.c_void_p]
        _lib.fmha_oracle_drop_threshold.argtypes = [C.c_float]
        _lib.fmha_oracle_drop_threshold.restype = C.c_uint32
        _lib.fmha_oracle_drop_scale.argtypes = [C.c_float]
        _lib.fmha_oracle_drop_scale.restype = C.c_float
        _lib.fmha_oracle_round.argtypes = [C.c_float, C.c_int]
        _lib.fmha_oracle_round.restype = C.c_float
    return _lib


ROUND = {None: 0, "none": 0, "fp32": 0, "fp16": 1, "half": 1, "bf16": 2, "e4m3": 3}


def _f32(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def philox4x32_10(ctr, key):
    """One Philox4x32-10 block: 4 counter words, 2 key words -> 4 output words."""
    c = np.asarray(ctr, dtype=np.uint32).copy()
    k = np.asarray(key, dtype=np.uint32).copy()
    out = np.zeros(4, dtype=np.uint32)
    lib().fmha_oracle_philox4x32_10(_ptr(c), _ptr(k), _ptr(out))
    return out


def round_to(x, kind):
    """Element-wise rounding of a float array to fp16 / bf16 / e4m3 (returned as float32)."""
    x = _f32(x)
    f = lib().fmha_oracle_round
    return np.array([f(float(v), ROUND[kind]) for v in x.ravel()], dtype=np.float32).reshape(x.shape)


def drop_threshold(p):
    return int(lib().fmha_oracle_drop_threshold(float(p)))


def drop_scale(p):
    """Factor on kept values: the reciprocal of the keep probability the 8-bit threshold realises."""
    return float(lib().fmha_oracle_drop_scale(float(p)))


def keep_mask(seed, offset, p, bh, sq, sk):
    """uint8 [bh,sq,sk] array of 0/1: the dropout keep decisions for (seed, offset)."""
    out = np.zeros((bh, sq, sk), dtype=np.uint8)
    lib().fmha_oracle_keep_mask(int(seed), int(offset), float(p), bh, sq, sk, _ptr(out))
    return out


def _mask_layout(mask, bh, sq, sk):
    """Normalise a mask of shape [bh,sq,sk], [bh,1,sk], [B,1,1,sk] or [B,1,sq,sk]."""
    m = _f32(mask)
    if m.ndim == 4:
        b = m.shape[0]
        assert m.shape[1] == 1 and bh % b == 0
        m = m.reshape(b, m.shape[2], m.shape[3])
    assert m.ndim == 3 and m.shape[2] == sk and bh % m.shape[0] == 0
    assert m.shape[1] in (1, sq)
    div = bh // m.shape[0]
    m_sq = 0 if m.shape[1] == 1 else sk
    m_sb = m.shape[1] * sk
    return m, div, m_sb, m_sq


def attention(q, k, v, mask=None, mask_kind="additive", mask_neg=-10000.0, causal=False,
              scale=None, drop_mask=None, drop_scale=None, p_drop=0.0, seed=0, offset=0,
              philox=False, round_p=None, round_o=None, dout=None, want=("o",), bh_offset=0):
    """Forward (and, when ``dout`` is given, backward) of the attention path on the CPU.

    ``drop_scale=None``: 1 with a dropout tensor, the mean-preserving factor ``drop_scale(p_drop)`` with Philox.
    ``bh_offset``: the tensors are heads ``bh_offset ..`` of a larger problem (Philox decisions follow).

    Returns a dict with the requested entries of
    ``o, lse, softmax, dropout, dq, dk, dv`` as float32 numpy arrays.
    """
    q, k, v = _f32(q), _f32(k), _f32(v)
    bh, sq, d = q.shape
    sk = k.shape[1]
    assert k.shape == (bh, sk, d) and v.shape == (bh, sk, d)
    P = _Params()
    P.bh, P.sq, P.sk, P.d = bh, sq, sk, d
    P.q, P.k, P.v = _ptr(q), _ptr(k), _ptr(v)
    keep = [q, k, v]
    if mask is not None:
        m, div, m_sb, m_sq = _mask_layout(mask, bh, sq, sk)
        keep.append(m)
        P.mask, P.mask_bh_div, P.mask_sb, P.mask_sq = _ptr(m), div, m_sb, m_sq
        P.mask_kind = {"additive": 1, "keep01": 2}[mask_kind]
    else:
        P.mask_bh_div = 1
    P.mask_neg = mask_neg
    P.causal = int(bool(causal))
    P.scale = float(scale) if scale is not None else 1.0 / np.sqrt(d)
    if drop_mask is not None:
        dm = _f32(drop_mask).reshape(bh, sq, sk)
        keep.append(dm)
        P.drop_kind, P.drop_mask = 1, _ptr(dm)
    elif philox:
        P.drop_kind = 2
        if drop_scale is None:
            drop_scale = globals()["drop_scale"](p_drop)
    if drop_scale is None:
        drop_scale = 1.0
    P.p_drop, P.drop_scale = float(p_drop), float(drop_scale)
    P.bh_offset = int(bh_offset)
    P.seed, P.offset = int(seed), int(offset)
    P.round_p, P.round_o = ROUND[round_p], ROUND[round_o]
    out = {}
    shapes = {"o": (bh, sq, d), "lse": (bh, sq), "softmax": (bh, sq, sk), "dropout": (bh, sq, sk),
              "dq": (bh, sq, d), "dk": (bh, sk, d), "dv": (bh, sk, d)}
    for name in want:
        out[name] = np.zeros(shapes[name], dtype=np.float32)
        setattr(P, name, _ptr(out[name]))
    if any(n in out for n in ("o", "lse", "softmax", "dropout")):
        rc = lib().fmha_oracle_fwd(C.byref(P))
        assert rc == 0
    if any(n in out for n in ("dq", "dk", "dv")):
        assert dout is not None
        do = _f32(dout)
        keep.append(do)
        P.dout = _ptr(do)
        rc = lib().fmha_oracle_bwd(C.byref(P))
        assert rc == 0
    return out
