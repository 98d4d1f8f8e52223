"""Row layouts other than the reference's folded [B*H, S, D]: the "permute" the reference leaves to
its callers (reference perf_measurement.py:52 labels its numbers "no permute"; fmha/fmha_manual.cpp
takes folded contiguous tensors only).  The kernels read [B, H, S, D] views of any batch / head /
row strides in place -- [B, S, H, D] memory, slices of a packed [B, S, 3, H, D] projection -- and
write their outputs in the same dimension order.

Checked against the CPU oracle on the same values (same tolerances as the other parity tests) and
bit for bit against this build's own folded path, which runs the same arithmetic.
"""
import numpy as np
import pytest
import torch

import oracle
from nvfuserexamples_amd import capi
from conftest import make_qkv, f32, rel_to_max, pad_mask

pytestmark = pytest.mark.gpu

TDT = {"fp16": torch.float16, "bf16": torch.bfloat16}
O_TOL = {"fp16": 2e-3, "bf16": 2e-2}
G_TOL = {"fp16": 1e-2, "bf16": 3e-2}


def _bshd(x, b, h):
    """[b*h, s, d] folded values -> [b, h, s, d] view of [b, s, h, d] memory."""
    bh, s, d = x.shape
    return x.view(b, h, s, d).permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)


def _packed(q, k, v, b, h):
    """Three [b, h, s, d] views into one packed [b, s, 3, h, d] buffer (needs sq == sk)."""
    bh, s, d = q.shape
    buf = torch.empty(b, s, 3, h, d, dtype=q.dtype, device=q.device)
    for i, x in enumerate((q, k, v)):
        buf[:, :, i] = x.view(b, h, s, d).permute(0, 2, 1, 3)
    return tuple(buf[:, :, i].permute(0, 2, 1, 3) for i in range(3))


CASES = [
    # b, h, sq, sk, d, dtype, causal, p_drop, mask, packed
    (2, 4, 128, 128, 64, "fp16", False, 0.0, False, False),
    (2, 3, 200, 333, 64, "fp16", False, 0.1, True, False),   # ragged tiles, dropout, padding mask
    (2, 3, 320, 320, 64, "fp16", True, 0.0, False, True),    # causal, packed projection
    (2, 2, 256, 256, 128, "bf16", True, 0.0, False, True),
    (40, 16, 128, 192, 64, "fp16", False, 0.0, True, False),  # more items than resident workgroups
    # short heads: the one-launch backward reads and writes the same layouts
    (3, 4, 197, 197, 64, "fp16", False, 0.1, False, True),    # ViT-B/16 length, packed projection
    (2, 3, 100, 128, 64, "bf16", True, 0.0, True, False),
    # head dim 256: plain forward loop, dQ kernel and the wave-pair dK/dV kernel on run-time row layouts
    (2, 2, 200, 264, 256, "fp16", False, 0.1, True, False),
    (2, 2, 192, 192, 256, "bf16", True, 0.0, False, True),
]


@pytest.mark.parametrize("b,h,sq,sk,d,dtype,causal,p,masked,packed", CASES)
def test_strided_layouts_match_oracle_and_folded_path(b, h, sq, sk, d, dtype, causal, p, masked, packed):
    bh = b * h
    q, k, v, do = make_qkv(bh, sq, sk, d, seed=bh + sk, std={64: 1.0, 128: 0.5, 256: 0.35}[d], dtype=dtype, with_dout=True)
    kw, okw = dict(causal=causal), dict(causal=causal)
    if p:
        kw.update(drop_kind=capi.DROP_PHILOX, p_drop=p, seed=11, offset=5)
        okw.update(philox=True, p_drop=p, seed=11, offset=5)
    m = None
    if masked:
        m = pad_mask(b, sk, sk // 2, sk).to(TDT[dtype])
        kw["mask"] = m.cuda()
    qc, kc, vc, doc = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    # folded path
    o3, l3, _, _ = capi.fwd(qc, kc, vc, want_lse=True, **kw)
    g3 = capi.bwd(doc, qc, kc, vc, o3, l3, **kw)
    # strided path on the same values
    if packed:
        q4, k4, v4 = _packed(qc, kc, vc, b, h)
    else:
        q4, k4, v4 = _bshd(qc, b, h), _bshd(kc, b, h), _bshd(vc, b, h)
    do4 = _bshd(doc, b, h)
    assert not q4.is_contiguous()
    o4, l4, _, _ = capi.fwd(q4, k4, v4, want_lse=True, **kw)
    g4 = capi.bwd(do4, q4, k4, v4, o4, l4, **kw)
    torch.cuda.synchronize()
    # outputs come back as [b, h, s, d] views of dense [b, s, h, d] memory
    for t in (o4, *g4):
        assert t.dim() == 4 and t.permute(0, 2, 1, 3).is_contiguous()
    assert l4.shape == (b, h, sq)
    assert torch.equal(o4.reshape(bh, sq, d), o3)
    assert torch.equal(l4.reshape(bh, sq), l3)
    for a4, a3 in zip(g4, g3):
        assert torch.equal(a4.reshape(a3.shape), a3)
    # and the folded values against the oracle
    mo = f32(m) if masked else None
    ref = oracle.attention(f32(q), f32(k), f32(v), mask=mo, dout=f32(do), want=("o", "dq", "dk", "dv"), **okw)
    assert np.abs(f32(o4.reshape(bh, sq, d).cpu()) - ref["o"]).max() <= O_TOL[dtype]
    for name, g in zip(("dq", "dk", "dv"), g4):
        assert rel_to_max(f32(g.reshape(ref[name].shape).cpu()), ref[name], floor=1e-3) <= G_TOL[dtype], name


def test_outputs_may_be_given_in_any_layout():
    b, h, s, d = 2, 4, 192, 64
    q, k, v = (t.cuda() for t in make_qkv(b * h, s, s, d, seed=4))
    o3, _, _, _ = capi.fwd(q, k, v)
    q4, k4, v4 = (t.view(b, h, s, d) for t in (q, k, v))       # contiguous [b, h, s, d]: the folded layout itself
    out = torch.empty(b, s, h, d, dtype=q.dtype, device="cuda").permute(0, 2, 1, 3)
    o4, _, _, _ = capi.fwd(q4, k4, v4, out=out)
    torch.cuda.synchronize()
    assert o4.data_ptr() == out.data_ptr()
    assert torch.equal(out.reshape(b * h, s, d), o3)
    # heads further apart than their rows need (a window of a longer buffer): only the head pitch differs
    wide = [torch.zeros(b, h, s + 8, d, dtype=q.dtype, device="cuda") for _ in range(3)]
    for w_, x in zip(wide, (q, k, v)):
        w_[:, :, :s] = x.view(b, h, s, d)
    o5, _, _, _ = capi.fwd(*(w_[:, :, :s] for w_ in wide))
    torch.cuda.synchronize()
    assert torch.equal(o5.reshape(b * h, s, d), o3)


def test_bad_strides_are_refused():
    b, h, s, d = 2, 2, 64, 64
    buf = torch.zeros(b, s, h, d + 4, dtype=torch.float16, device="cuda")  # rows 68 elements apart
    x = buf[..., :d].permute(0, 2, 1, 3)
    with pytest.raises(capi.FmhaError):
        capi.fwd(x, x, x)
    k = torch.zeros(b, h, s, d, dtype=torch.float16, device="cuda")
    v = torch.zeros(b, s, h, d, dtype=torch.float16, device="cuda").permute(0, 2, 1, 3)
    with pytest.raises(capi.FmhaError):   # k and v rows must be equally far apart
        capi.fwd(k, k, v)
    q3 = torch.zeros(b * h, s, d, dtype=torch.float16, device="cuda")
    with pytest.raises(capi.FmhaError):   # folded and 4-d tensors do not mix
        capi.fwd(q3, k, k)


def test_operators_and_autograd_take_strided_tensors():
    from nvfuserexamples_amd import load_ops
    from nvfuserexamples_amd.autograd import attention
    ops = load_ops()
    b, h, s, d = 2, 4, 256, 64
    q, k, v, do = (t.cuda() for t in make_qkv(b * h, s, s, d, seed=8, with_dout=True))
    m = pad_mask(b, s, s // 2, s).half().cuda()
    o3, l3 = ops.fmha_fwd(q, k, v, m, 0.0, False, 0.1, 7, 3)
    g3 = ops.fmha_bwd(do, q, k, v, o3, l3, m, 0.0, False, 0.1, 7, 3)
    q4, k4, v4 = _packed(q, k, v, b, h)
    do4 = _bshd(do, b, h)
    o4, l4 = ops.fmha_fwd(q4, k4, v4, m, 0.0, False, 0.1, 7, 3)
    g4 = ops.fmha_bwd(do4, q4, k4, v4, o4, l4, m, 0.0, False, 0.1, 7, 3)
    assert o4.shape == (b, h, s, d) and o4.permute(0, 2, 1, 3).is_contiguous() and l4.shape == (b, h, s)
    assert torch.equal(o4.reshape(b * h, s, d), o3)
    for a4, a3 in zip(g4, g3):
        assert torch.equal(a4.reshape(a3.shape), a3)
    # a row pitch the kernels cannot read in place is copied by the operator, not refused
    buf = torch.zeros(b, s, h, d + 4, dtype=torch.float16, device="cuda")
    buf[..., :d] = q.view(b, h, s, d).permute(0, 2, 1, 3)
    o5, _ = ops.fmha_fwd(buf[..., :d].permute(0, 2, 1, 3), k4, v4, m, 0.0, False, 0.1, 7, 3)
    assert torch.equal(o5.reshape(b * h, s, d), o3)
    # so are K and V whose rows are not equally far apart
    o6, _ = ops.fmha_fwd(q4, k.view(b, h, s, d), v4, m, 0.0, False, 0.1, 7, 3)
    assert torch.equal(o6.reshape(b * h, s, d), o3)
    # autograd through a packed projection: gradients land in the packed buffer's layout
    packed = torch.empty(b, s, 3, h, d, dtype=torch.float16, device="cuda")
    for i, x in enumerate((q, k, v)):
        packed[:, :, i] = x.view(b, h, s, d).permute(0, 2, 1, 3)
    packed.requires_grad_(True)
    qa, ka, va = (packed[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    oa = attention(qa, ka, va, mask=m, p_drop=0.1, seed=7, offset=3)
    oa.backward(do4)
    gp = packed.grad
    for i, a3 in enumerate(g3):
        assert torch.equal(gp[:, :, i].permute(0, 2, 1, 3).reshape(a3.shape), a3)


def test_headline_shape_packed_projection_equals_folded_path(monkeypatch):
    """B32 H16 S512 D64 with a padding mask, read from a packed [B,S,3,H,D] buffer: at this shape the
    pipelined forward deals the mask rows to its workgroups by length, in both layouts alike.  Full size, so the
    check is bit-equality with the folded path on the same kernel (itself held to the oracle elsewhere), train
    step included.  (By default the folded layout takes the whole-head kernel at this shape, which walks the keys
    in tiles of 32 instead of 64: its output agrees to the rounding of the element type, not bit for bit.)"""
    b, h, s, d = 32, 16, 512, 64
    q, k, v, do = make_qkv(b * h, s, s, d, seed=21, with_dout=True)
    kw = dict(mask=pad_mask(b, s, s // 2, s).half().cuda(), drop_kind=capi.DROP_PHILOX, p_drop=0.1, seed=3, offset=9)
    qc, kc, vc, doc = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    o_head, l_head, _, _ = capi.fwd(qc, kc, vc, want_lse=True, **kw)
    monkeypatch.setenv("FMHA_FWD_HEAD", "0")
    o3, l3, _, _ = capi.fwd(qc, kc, vc, want_lse=True, **kw)
    assert (o_head.float() - o3.float()).abs().max().item() <= 2e-3
    assert (l_head - l3).abs().max().item() <= 1e-3
    g3 = capi.bwd(doc, qc, kc, vc, o3, l3, **kw)
    q4, k4, v4 = _packed(qc, kc, vc, b, h)
    o4, l4, _, _ = capi.fwd(q4, k4, v4, want_lse=True, **kw)
    g4 = capi.bwd(_bshd(doc, b, h), q4, k4, v4, o4, l4, **kw)
    torch.cuda.synchronize()
    assert torch.equal(o4.reshape(b * h, s, d), o3)
    assert torch.equal(l4.reshape(b * h, s), l3)
    for a4, a3 in zip(g4, g3):
        assert torch.equal(a4.reshape(a3.shape), a3)
    # and without the dealing and the trimming
    o0 = capi.fwd(q4, k4, v4, flags=capi.FLAG_NO_MASK_TRIM, **kw)[0]
    assert torch.equal(o0, o4)
    # the whole-head kernel reads the packed buffer in place too, and gives the bits it gives on folded tensors
    monkeypatch.delenv("FMHA_FWD_HEAD")
    o5, l5, _, _ = capi.fwd(q4, k4, v4, want_lse=True, **kw)
    torch.cuda.synchronize()
    assert torch.equal(o5.reshape(b * h, s, d), o_head)
    assert torch.equal(l5.reshape(b * h, s), l_head)


@pytest.mark.parametrize("b,h,sq,sk,p,masked,packed", [
    (2, 3, 200, 333, 0.1, True, False),    # ragged query chunk, partly filled last key tile, dropout, padding mask
    (3, 2, 512, 264, 0.0, False, True),    # packed projection, no mask
    (1, 4, 1030, 512, 0.3, True, True),    # three 512-query items per head, the last one nearly empty
])
def test_whole_head_kernel_on_strided_layouts(b, h, sq, sk, p, masked, packed, monkeypatch):
    """FMHA_FWD_HEAD=1 puts every eligible forward on the whole-head kernel: [B,H,S,D] views of [B,S,H,D] memory and
    slices of a packed projection against the folded tensors (same bits) and the oracle."""
    monkeypatch.setenv("FMHA_FWD_HEAD", "1")
    bh, d = b * h, 64
    q, k, v = make_qkv(bh, sq, sk, d, seed=bh + sk)
    if packed and sq != sk:
        packed = False   # (one packed buffer holds q, k and v of one length)
    kw, okw = {}, {}
    if p:
        kw.update(drop_kind=capi.DROP_PHILOX, p_drop=p, seed=11, offset=5)
        okw.update(philox=True, p_drop=p, seed=11, offset=5)
    m = None
    if masked:
        m = pad_mask(b, sk, sk // 2, sk).half()
        kw["mask"] = m.cuda()
    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    o3, l3, _, _ = capi.fwd(qc, kc, vc, want_lse=True, **kw)
    if packed:
        q4, k4, v4 = _packed(qc, kc, vc, b, h)
    else:
        q4, k4, v4 = _bshd(qc, b, h), _bshd(kc, b, h), _bshd(vc, b, h)
    o4, l4, _, _ = capi.fwd(q4, k4, v4, want_lse=True, **kw)
    torch.cuda.synchronize()
    assert o4.permute(0, 2, 1, 3).is_contiguous()
    assert torch.equal(o4.reshape(bh, sq, d), o3)
    assert torch.equal(l4.reshape(bh, sq), l3)
    ref = oracle.attention(f32(q), f32(k), f32(v), mask=f32(m) if masked else None, want=("o", "lse"), **okw)
    assert np.abs(f32(o4.reshape(bh, sq, d).cpu()) - ref["o"]).max() <= O_TOL["fp16"]
    assert np.abs(l4.reshape(bh, sq).cpu().numpy() - ref["lse"]).max() <= 1e-3
