"""ctypes binding of ``libfmha_hip.so`` (the C ABI declared in ``include/fmha_capi.h``).

This is the thinnest possible host layer: torch is used only for device memory and
the current HIP stream.  There is no CPU fallback -- if the library is missing the
import of :func:`lib` raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libfmha_hip.so")

F16, BF16 = 0, 1
MASK_NONE, MASK_ADDITIVE, MASK_KEEP01 = 0, 1, 2
FLAG_NO_MASK_TRIM = 1  # fwd(flags=...): visit every key tile even where a per-key mask hard-masks the tail
DROP_NONE, DROP_PHILOX, DROP_TENSOR = 0, 1, 2

EXPORTS = ("fmha_fwd_launch", "fmha_bwd_launch", "fmha_bwd_workspace_bytes", "fmha_philox_keep_mask",
           "fmha_drop_threshold", "fmha_strerror", "fmha_version", "fmha_reload_overrides",
           "fmha_bwd_launch_noalloc", "fmha_bwd_noalloc_max_rows", "fmha_drop_scale", "fmha_fwd_fp8_launch",
           "fmha_fwd_workspace_bytes", "fmha_fwd_fp8_workspace_bytes", "fmha_pipe_probe")
# environment overrides the library reads once; the wrappers below make it read them again when they change
_ENV_NAMES = ("FMHA_MASK_TRIM", "FMHA_FWD_SHORT", "FMHA_FWD_SAVE_SPLIT", "FMHA_FWD_SAVE_ONCE", "FMHA_FWD_STREAM", "FMHA_FWD_QB", "FMHA_FWD_SPLIT", "FMHA_FWD_DECODE", "FMHA_FWD_HEAD",
              "FMHA_BWD_PAIR", "FMHA_BWD_SHORT")
_env_seen = None


def _sync_env():
    global _env_seen
    now = tuple(os.environ.get(n) for n in _ENV_NAMES)
    if now != _env_seen:
        lib().fmha_reload_overrides()
        _env_seen = now


class _Params(C.Structure):
    """Parameter structs carry their own size first (the library reads that many bytes)."""

    def __init__(self, *args, **kw):
        super().__init__(*args, **kw)
        self.struct_bytes = C.sizeof(self)


class FwdParams(_Params):
    _fields_ = [
        ("struct_bytes", C.c_uint64),
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("o", C.c_void_p), ("lse", C.c_void_p),
        ("mask", C.c_void_p), ("mask_kind", C.c_int32), ("causal", C.c_int32),
        ("mask_bh_div", C.c_int64), ("mask_stride_b", C.c_int64), ("mask_stride_q", C.c_int64),
        ("mask_neg", C.c_float),
        ("drop_kind", C.c_int32), ("drop_mask", C.c_void_p), ("p_drop", C.c_float), ("drop_scale", C.c_float),
        ("seed", C.c_uint64), ("offset", C.c_uint64),
        ("save_softmax", C.c_void_p), ("save_dropout", C.c_void_p),
        ("bh", C.c_int32), ("sq", C.c_int32), ("sk", C.c_int32), ("d", C.c_int32),
        ("dtype", C.c_int32), ("scale", C.c_float), ("flags", C.c_int32),
        ("kv_len", C.c_void_p), ("kv_len_bh_div", C.c_int32),
        ("clock_probe", C.c_void_p),
        ("heads", C.c_int32),
        ("q_stride", C.c_int64 * 3), ("k_stride", C.c_int64 * 3), ("v_stride", C.c_int64 * 3),
        ("o_stride", C.c_int64 * 3),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_uint64),
    ]


class BwdParams(_Params):
    _fields_ = [
        ("struct_bytes", C.c_uint64),
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("o", C.c_void_p), ("dout", C.c_void_p),
        ("lse", C.c_void_p), ("delta", C.c_void_p),
        ("dq", C.c_void_p), ("dk", C.c_void_p), ("dv", C.c_void_p),
        ("mask", C.c_void_p), ("mask_kind", C.c_int32), ("causal", C.c_int32),
        ("mask_bh_div", C.c_int64), ("mask_stride_b", C.c_int64), ("mask_stride_q", C.c_int64),
        ("mask_neg", C.c_float),
        ("drop_kind", C.c_int32), ("drop_mask", C.c_void_p), ("p_drop", C.c_float), ("drop_scale", C.c_float),
        ("seed", C.c_uint64), ("offset", C.c_uint64),
        ("bh", C.c_int32), ("sq", C.c_int32), ("sk", C.c_int32), ("d", C.c_int32),
        ("dtype", C.c_int32), ("scale", C.c_float), ("flags", C.c_int32),
        ("kv_len", C.c_void_p), ("kv_len_bh_div", C.c_int32),
        ("heads", C.c_int32),
        ("q_stride", C.c_int64 * 3), ("k_stride", C.c_int64 * 3), ("v_stride", C.c_int64 * 3),
        ("o_stride", C.c_int64 * 3), ("do_stride", C.c_int64 * 3),
        ("dq_stride", C.c_int64 * 3), ("dk_stride", C.c_int64 * 3), ("dv_stride", C.c_int64 * 3),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_uint64),
    ]


class FwdFp8Params(_Params):
    _fields_ = [
        ("struct_bytes", C.c_uint64),
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("o", C.c_void_p), ("lse", C.c_void_p),
        ("mask", C.c_void_p), ("mask_bh_div", C.c_int64), ("mask_stride_b", C.c_int64),
        ("bh", C.c_int32), ("sq", C.c_int32), ("sk", C.c_int32), ("d", C.c_int32),
        ("out_dtype", C.c_int32),
        ("scale", C.c_float), ("descale_q", C.c_float), ("descale_k", C.c_float), ("descale_v", C.c_float),
        ("causal", C.c_int32),
        ("kv_len", C.c_void_p), ("kv_len_bh_div", C.c_int32),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_uint64),
    ]


class FmhaError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"fmha error {code}: {msg}")
        self.code = code


_lib = None


def lib():
    """Load the shared library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m nvfuserexamples_amd.build` "
                "(there is no fallback path)")
        L = C.CDLL(LIB_PATH)
        L.fmha_fwd_launch.argtypes = [C.POINTER(FwdParams), C.c_void_p]
        L.fmha_fwd_launch.restype = C.c_int
        L.fmha_fwd_workspace_bytes.argtypes = [C.POINTER(FwdParams)]
        L.fmha_fwd_workspace_bytes.restype = C.c_uint64
        L.fmha_bwd_launch.argtypes = [C.POINTER(BwdParams), C.c_void_p]
        L.fmha_bwd_launch.restype = C.c_int
        L.fmha_fwd_fp8_launch.argtypes = [C.POINTER(FwdFp8Params), C.c_void_p]
        L.fmha_fwd_fp8_launch.restype = C.c_int
        L.fmha_fwd_fp8_workspace_bytes.argtypes = [C.POINTER(FwdFp8Params)]
        L.fmha_fwd_fp8_workspace_bytes.restype = C.c_uint64
        L.fmha_bwd_launch_noalloc.argtypes = [C.POINTER(BwdParams), C.c_void_p]
        L.fmha_bwd_launch_noalloc.restype = C.c_int
        L.fmha_bwd_noalloc_max_rows.argtypes = []
        L.fmha_bwd_noalloc_max_rows.restype = C.c_uint64
        L.fmha_bwd_workspace_bytes.argtypes = [C.c_int32, C.c_int32, C.c_int32, C.c_int32]
        L.fmha_bwd_workspace_bytes.restype = C.c_uint64
        L.fmha_philox_keep_mask.argtypes = [C.c_uint64, C.c_uint64, C.c_float, C.c_int32, C.c_int32,
                                            C.c_int32, C.c_void_p, C.c_void_p]
        L.fmha_philox_keep_mask.restype = C.c_int
        L.fmha_drop_threshold.argtypes = [C.c_float]
        L.fmha_drop_threshold.restype = C.c_uint32
        L.fmha_drop_scale.argtypes = [C.c_float]
        L.fmha_drop_scale.restype = C.c_float
        L.fmha_strerror.argtypes = [C.c_int]
        L.fmha_strerror.restype = C.c_char_p
        L.fmha_version.restype = C.c_char_p
        L.fmha_pipe_probe.argtypes = [C.c_int] * 6 + [C.POINTER(C.c_double)]
        L.fmha_pipe_probe.restype = C.c_int
        L.fmha_reload_overrides.argtypes = []
        L.fmha_reload_overrides.restype = None
        _lib = L
    return _lib


def check(rc):
    if rc != 0:
        raise FmhaError(rc, lib().fmha_strerror(rc).decode())


def _dtype_code(t):
    import torch
    if t.dtype == torch.float16:
        return F16
    if t.dtype == torch.bfloat16:
        return BF16
    raise FmhaError(-2, "tensors must be float16 or bfloat16")


def _stream_ptr():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def mask_layout(mask, bh, sq, sk):
    """(bh_div, stride_b, stride_q) of a mask shaped [bh,sq,sk], [bh,1,sk], [B,1,1,sk] or [B,1,sq,sk]."""
    if mask.dim() == 4:
        if mask.shape[1] != 1:
            raise FmhaError(-5, "4-d masks must be [B,1,sq|1,sk]")
        mask = mask.reshape(mask.shape[0], mask.shape[2], mask.shape[3])
    if mask.dim() != 3 or mask.shape[2] != sk or mask.shape[1] not in (1, sq) or bh % mask.shape[0]:
        raise FmhaError(-5, f"mask shape {tuple(mask.shape)} does not broadcast over [{bh},{sq},{sk}]")
    if not mask.is_contiguous():
        raise FmhaError(-5, "mask must be contiguous")
    div = bh // mask.shape[0]
    return mask, div, mask.shape[1] * sk, (0 if mask.shape[1] == 1 else sk)


def _set_kv_len(P, kv_len, bh):
    import torch
    if kv_len is None:
        return
    if not (kv_len.is_cuda and kv_len.is_contiguous() and kv_len.dtype == torch.int32 and kv_len.dim() == 1
            and kv_len.numel() > 0 and bh % kv_len.numel() == 0):
        raise FmhaError(-5, "kv_len must be a contiguous int32 device vector whose length divides bh")
    P.kv_len, P.kv_len_bh_div = kv_len.data_ptr(), bh // kv_len.numel()


def _rows(t, name):
    """(bh, rows, d, heads, strides) of a [bh, rows, d] contiguous or a [B, H, rows, d] strided tensor."""
    if t.dim() == 3:
        if not t.is_contiguous():
            raise FmhaError(-5, f"{name}: 3-d tensors must be contiguous [bh, s, d]; pass a 4-d [B, H, s, d] view for other layouts")
        return t.shape[0], t.shape[1], t.shape[2], 0, (0, 0, 0)
    if t.dim() != 4 or t.stride(3) != 1:
        raise FmhaError(-5, f"{name} must be [bh, s, d] or [B, H, s, d] with contiguous rows")
    return t.shape[0] * t.shape[1], t.shape[2], t.shape[3], t.shape[1], (t.stride(0), t.stride(1), t.stride(2))


def empty_like_rows(t):
    """New tensor of t's shape whose dimensions are laid out in t's order but densely (a slice
    of a packed [B, s, 3, H, d] tensor gives a [B, H, s, d] view of fresh [B, s, H, d] memory)."""
    import torch
    if t.dim() == 3:
        return torch.empty_like(t)
    order = sorted(range(4), key=lambda i: (-t.stride(i), i))
    base = torch.empty([t.shape[i] for i in order], dtype=t.dtype, device=t.device)
    inv = [order.index(i) for i in range(4)]
    return base.permute(inv)


def _set_rows(P, heads, **tensors):
    """Fill P.heads and P.<name>_stride; all tensors must agree on 3-d (folded) or 4-d with one H."""
    hs = {h for _, h, _ in tensors.values()}
    if len(hs) != 1:
        raise FmhaError(-5, "tensors must be all [bh, s, d] or all [B, H, s, d] with the same H")
    P.heads = heads
    for name, (_, _, st) in tensors.items():
        arr = getattr(P, name + "_stride")
        for i in range(3):
            arr[i] = st[i]


def fwd(q, k, v, mask=None, mask_kind=MASK_ADDITIVE, mask_neg=-10000.0, causal=False, scale=None,
        drop_kind=DROP_NONE, drop_mask=None, p_drop=0.0, drop_scale=None, seed=0, offset=0,
        want_lse=False, save=False, flags=0, out=None, kv_len=None, workspace=True):
    """Launch the forward on the current stream.  Returns (o, lse|None, softmax|None, dropout|None).

    workspace: True allocates what ``fmha_fwd_workspace_bytes`` asks for (nothing for most shapes: only
    launches with few heads, few query rows and a long key range run their key range in pieces), False
    passes none (always the plain launch), a uint8 device tensor is passed as it is.

    kv_len: optional int32 device tensor of B valid key counts (bh must be a multiple of B); head i
    attends keys [0, kv_len[i // (bh // B)]) only.

    q, k, v: contiguous [bh, s, d] (the reference's layout), or 4-d [B, H, s, d] tensors with
    arbitrary batch / head / row strides (multiples of 8 elements; rows contiguous), e.g.
    ``x.view(B, s, H, d).transpose(1, 2)`` or a slice of a packed QKV projection: no copy is made.
    o then comes back as [B, H, sq, d] in q's dimension order and lse as [B, H, sq]."""
    import torch
    bh, sq, d, heads, qs = _rows(q, "q")
    bhk, sk, dk_, hk, ks = _rows(k, "k")
    bhv, skv, dv_, hv, vs = _rows(v, "v")
    if (bhk, dk_, bhv, skv, dv_) != (bh, d, bh, sk, d):
        raise FmhaError(-3, "q/k/v shapes do not agree")
    P = FwdParams()
    P.dtype = _dtype_code(q)
    for t in (q, k, v):
        if not (t.is_cuda and t.dtype == q.dtype):
            raise FmhaError(-5, "q/k/v must be device tensors of one dtype")
    o = out if out is not None else empty_like_rows(q)
    _, _, _, ho, os_ = _rows(o, "out")
    _set_rows(P, heads, q=(0, heads, qs), k=(0, hk, ks), v=(0, hv, vs), o=(0, ho, os_))
    lse = torch.empty((bh, sq) if heads == 0 else (q.shape[0], heads, sq), dtype=torch.float32,
                      device=q.device) if want_lse else None
    P.q, P.k, P.v, P.o = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr()
    P.lse = lse.data_ptr() if lse is not None else None
    lse_scratch = None
    if save and lse is None:   # with an LSE buffer the library takes the faster route to the saved outputs
        lse_scratch = torch.empty((bh, sq), dtype=torch.float32, device=q.device)
        P.lse = lse_scratch.data_ptr()
    P.bh, P.sq, P.sk, P.d = bh, sq, sk, d
    P.scale = float(scale) if scale is not None else d ** -0.5
    P.causal = int(bool(causal))
    P.mask_neg = mask_neg
    if mask is not None:
        mask, div, sb, sqs = mask_layout(mask, bh, sq, sk)
        if mask.dtype != q.dtype:
            raise FmhaError(-5, "mask dtype must match q")
        P.mask, P.mask_kind = mask.data_ptr(), mask_kind
        P.mask_bh_div, P.mask_stride_b, P.mask_stride_q = div, sb, sqs
    P.drop_kind = drop_kind
    if drop_kind == DROP_TENSOR:
        if drop_mask is None or drop_mask.dtype != q.dtype or not drop_mask.is_contiguous():
            raise FmhaError(-5, "drop_mask must be a contiguous tensor of q's dtype")
        P.drop_mask = drop_mask.data_ptr()
    P.p_drop = p_drop
    if drop_scale is None:   # Philox: the factor that keeps the mean at the realised keep probability
        drop_scale = lib().fmha_drop_scale(p_drop) if drop_kind == DROP_PHILOX else 1.0
    P.drop_scale = drop_scale
    P.seed, P.offset = seed, offset
    sm = dr = None
    if save:
        sm = torch.empty((bh, sq, sk), dtype=q.dtype, device=q.device)
        dr = torch.empty((bh, sq, sk), dtype=q.dtype, device=q.device)
        P.save_softmax, P.save_dropout = sm.data_ptr(), dr.data_ptr()
    P.flags = flags
    _set_kv_len(P, kv_len, bh)
    _sync_env()
    ws = None
    if workspace is True:
        need = lib().fmha_fwd_workspace_bytes(C.byref(P))
        if need:
            ws = torch.empty(need, dtype=torch.uint8, device=q.device)
    elif workspace is not False and workspace is not None:
        ws = workspace
    if ws is not None:
        P.workspace, P.workspace_bytes = ws.data_ptr(), ws.numel()
    check(lib().fmha_fwd_launch(C.byref(P), _stream_ptr()))
    return o, lse, sm, dr


def bwd(dout, q, k, v, o, lse, mask=None, mask_kind=MASK_ADDITIVE, mask_neg=-10000.0, causal=False,
        scale=None, drop_kind=DROP_NONE, drop_mask=None, p_drop=0.0, drop_scale=None, seed=0, offset=0,
        flags=0, delta=None, grads=None, kv_len=None, workspace=True, noalloc=False):
    """Launch the backward on the current stream.  Returns (dq, dk, dv).  kv_len and the tensor
    layouts as in fwd(); each gradient comes back in its input's dimension order.

    workspace: True allocates the scratch that fmha_bwd_workspace_bytes() asks for (none: no backward kernel uses one), a uint8
    device tensor is passed on as it is, None / False passes none (the two-kernel path beyond 256 keys).
    noalloc: call fmha_bwd_launch_noalloc (delta out of the library's own scratch memory)."""
    import torch
    bh, sq, d, heads, qs = _rows(q, "q")
    _, sk, _, hk, ks = _rows(k, "k")
    _, _, _, hv, vs = _rows(v, "v")
    _, _, _, ho, os_ = _rows(o, "o")
    _, _, _, hd, ds_ = _rows(dout, "dout")
    if not (k.shape == v.shape and o.shape == q.shape and dout.shape == q.shape and k.shape[-1] == d):
        raise FmhaError(-3, "q/k/v/o/dout shapes do not agree")
    P = BwdParams()
    P.dtype = _dtype_code(q)
    for t in (q, k, v, o, dout):
        if not (t.is_cuda and t.dtype == q.dtype):
            raise FmhaError(-5, "q/k/v/o/dout must be device tensors of one dtype")
    if delta is None and not noalloc:
        delta = torch.empty((bh, sq), dtype=torch.float32, device=q.device)
    if not lse.is_contiguous():
        raise FmhaError(-5, "lse must be contiguous")
    dq, dk, dv = grads if grads is not None else (empty_like_rows(q), empty_like_rows(k), empty_like_rows(v))
    _set_rows(P, heads, q=(0, heads, qs), k=(0, hk, ks), v=(0, hv, vs), o=(0, ho, os_), do=(0, hd, ds_),
              dq=(0,) + _rows(dq, "dq")[3:], dk=(0,) + _rows(dk, "dk")[3:], dv=(0,) + _rows(dv, "dv")[3:])
    P.q, P.k, P.v, P.o, P.dout = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), dout.data_ptr()
    P.lse, P.delta = lse.data_ptr(), (None if noalloc else delta.data_ptr())
    P.dq, P.dk, P.dv = dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    P.bh, P.sq, P.sk, P.d = bh, sq, sk, d
    P.scale = float(scale) if scale is not None else d ** -0.5
    P.causal = int(bool(causal))
    P.mask_neg = mask_neg
    if mask is not None:
        mask, div, sb, sqs = mask_layout(mask, bh, sq, sk)
        P.mask, P.mask_kind = mask.data_ptr(), mask_kind
        P.mask_bh_div, P.mask_stride_b, P.mask_stride_q = div, sb, sqs
    P.drop_kind = drop_kind
    if drop_kind == DROP_TENSOR:
        P.drop_mask = drop_mask.data_ptr()
    P.p_drop = p_drop
    if drop_scale is None:   # Philox: the factor that keeps the mean at the realised keep probability
        drop_scale = lib().fmha_drop_scale(p_drop) if drop_kind == DROP_PHILOX else 1.0
    P.drop_scale = drop_scale
    P.seed, P.offset = seed, offset
    P.flags = flags
    _set_kv_len(P, kv_len, bh)
    if noalloc:
        _sync_env()
        check(lib().fmha_bwd_launch_noalloc(C.byref(P), _stream_ptr()))
        return dq, dk, dv
    if workspace is True:
        need = lib().fmha_bwd_workspace_bytes(bh, sq, sk, d)
        workspace = torch.empty(need, dtype=torch.uint8, device=q.device) if need else None
    if workspace is not None and workspace is not False:
        P.workspace, P.workspace_bytes = workspace.data_ptr(), workspace.numel() * workspace.element_size()
    _sync_env()
    check(lib().fmha_bwd_launch(C.byref(P), _stream_ptr()))
    return dq, dk, dv


def fwd_fp8(q8, k8, v8, descale_q=1.0, descale_k=1.0, descale_v=1.0, mask=None, causal=False, scale=None,
            out_dtype=None, want_lse=False, kv_len=None, workspace=True):
    """Forward on e4m3 inputs (torch.float8_e4m3fn, contiguous [bh, s, d]) on the current stream.
    Returns (o, lse|None); o is float16 unless out_dtype says bfloat16.  mask: additive [bh|B, 1, sk] /
    [B,1,1,sk] in o's dtype.  kv_len (valid key counts, as in fwd) and workspace (as in fwd) apply to launches
    of one to four query rows without a causal mask, which run on the streaming decode kernel."""
    import torch
    out_dtype = out_dtype or torch.float16
    for t in (q8, k8, v8):
        if not (t.is_cuda and t.dtype == torch.float8_e4m3fn and t.dim() == 3 and t.is_contiguous()):
            raise FmhaError(-5, "q, k, v must be contiguous [bh, s, d] float8_e4m3fn device tensors")
    bh, sq, d = q8.shape
    sk = k8.shape[1]
    if k8.shape != (bh, sk, d) or v8.shape != (bh, sk, d):
        raise FmhaError(-3, "q/k/v shapes do not agree")
    P = FwdFp8Params()
    o = torch.empty((bh, sq, d), dtype=out_dtype, device=q8.device)
    lse = torch.empty((bh, sq), dtype=torch.float32, device=q8.device) if want_lse else None
    P.q, P.k, P.v, P.o = q8.data_ptr(), k8.data_ptr(), v8.data_ptr(), o.data_ptr()
    P.lse = lse.data_ptr() if lse is not None else None
    P.bh, P.sq, P.sk, P.d = bh, sq, sk, d
    P.out_dtype = F16 if out_dtype == torch.float16 else BF16
    P.scale = float(scale) if scale is not None else d ** -0.5
    P.descale_q, P.descale_k, P.descale_v = descale_q, descale_k, descale_v
    P.causal = int(bool(causal))
    if mask is not None:
        mask, div, sb, sqs = mask_layout(mask, bh, sq, sk)
        if mask.dtype != out_dtype or sqs != 0:
            raise FmhaError(-5, "the e4m3 forward takes a per-key mask ([.., 1, sk]) of o's dtype")
        P.mask, P.mask_bh_div, P.mask_stride_b = mask.data_ptr(), div, sb
    _set_kv_len(P, kv_len, bh)
    _sync_env()
    ws = None
    if workspace is True:
        need = lib().fmha_fwd_fp8_workspace_bytes(C.byref(P))
        if need:
            ws = torch.empty(need, dtype=torch.uint8, device=q8.device)
    elif workspace is not False and workspace is not None:
        ws = workspace
    if ws is not None:
        P.workspace, P.workspace_bytes = ws.data_ptr(), ws.numel()
    check(lib().fmha_fwd_fp8_launch(C.byref(P), _stream_ptr()))
    return o, lse


def philox_keep_mask(seed, offset, p_drop, bh, sq, sk, device="cuda"):
    """uint8 [bh,sq,sk] device tensor of the keep decisions the kernels use."""
    import torch
    out = torch.empty((bh, sq, sk), dtype=torch.uint8, device=device)
    check(lib().fmha_philox_keep_mask(seed, offset, p_drop, bh, sq, sk, out.data_ptr(), _stream_ptr()))
    return out
