"""fmha_bwd_launch_noalloc (delta and workspace out of the library's own device array) against
fmha_bwd_launch on the same inputs, through the C ABI: bit-identical gradients, on two calls in a row,
the second with a smaller input (the array keeps the first call's contents)."""
import ctypes as C

import pytest
import torch

from nvfuserexamples_amd import capi
from conftest import make_qkv, pad_mask

pytestmark = pytest.mark.gpu


def _params(q, k, v, o, do, lse, mask, dq, dk, dv, delta, flags=0):
    bh, sq, d = q.shape
    P = capi.BwdParams()
    P.q, P.k, P.v, P.o, P.dout = (t.data_ptr() for t in (q, k, v, o, do))
    P.lse = lse.data_ptr()
    P.delta = delta.data_ptr() if delta is not None else None
    P.dq, P.dk, P.dv = dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    P.bh, P.sq, P.sk, P.d = bh, sq, k.shape[1], d
    P.dtype = capi.F16
    P.scale = d ** -0.5
    P.mask, P.mask_kind = mask.data_ptr(), capi.MASK_ADDITIVE
    P.mask_bh_div, P.mask_stride_b, P.mask_stride_q = bh // mask.shape[0], k.shape[1], 0
    P.drop_kind, P.p_drop, P.drop_scale, P.seed, P.offset = capi.DROP_PHILOX, 0.1, 0.0, 5, 7  # scale 0: the mean-preserving factor
    P.flags = flags
    return P


def _both_ways(bh, sq, sk, seed, flags=0):
    L = capi.lib()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    q, k, v, do = (t.cuda() for t in make_qkv(bh, sq, sk, 64, seed=seed, with_dout=True))
    m = pad_mask(bh // 2, sk, sk // 2, sk).half().cuda()
    o, lse, _, _ = capi.fwd(q, k, v, mask=m, want_lse=True, drop_kind=capi.DROP_PHILOX, p_drop=0.1, seed=5, offset=7)
    ref = [torch.empty_like(t) for t in (q, k, v)]
    delta = torch.empty(bh, sq, dtype=torch.float32, device="cuda")
    P = _params(q, k, v, o, do, lse, m, *ref, delta, flags)
    capi.check(L.fmha_bwd_launch(C.byref(P), stream))
    got = [torch.full_like(t, float("nan")) for t in (q, k, v)]
    Pn = _params(q, k, v, o, do, lse, m, *got, None, flags)
    capi.check(L.fmha_bwd_launch_noalloc(C.byref(Pn), stream))
    torch.cuda.synchronize()
    for a, b in zip(got, ref):
        assert torch.equal(a, b)
    assert all(torch.isfinite(t.float()).all() for t in got)


def test_noalloc_backward_equals_the_allocating_entry_point_twice_in_a_row():
    _both_ways(8, 512, 512, seed=1)
    _both_ways(4, 200, 333, seed=2)     # smaller, over what the first call left in the array


def test_noalloc_backward_refuses_what_does_not_fit():
    L = capi.lib()
    rows = int(L.fmha_bwd_noalloc_max_rows())
    assert rows == 2 * 1024 * 1024
    bh, sq = 4100, 512                   # 2 099 200 rows
    assert bh * sq > rows
    q = torch.empty(1, device="cuda", dtype=torch.float16)
    P = capi.BwdParams()
    for n in ("q", "k", "v", "o", "dout", "lse", "dq", "dk", "dv"):
        setattr(P, n, q.data_ptr())
    P.bh, P.sq, P.sk, P.d, P.dtype, P.scale = bh, sq, 512, 64, capi.F16, 0.125
    rc = L.fmha_bwd_launch_noalloc(C.byref(P), None)
    assert rc == -8 and b"fmha_bwd_noalloc_max_rows" in L.fmha_strerror(rc)
