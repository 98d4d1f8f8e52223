"""Head dims other than the three the kernels are built for (64, 128 and 256).

The reference is fixed at D = 64 (fmha/fmha_manual.cpp:39-47).  The C ABI takes any multiple of 8 up
to 256: the kernels run at the next built size and neither read nor write the columns a row does not
have (no padded copies anywhere).  The general operators also take head dims that are not multiples of
8, by zero-padding to the next multiple.  Zero columns change neither Q.K^T nor the kept columns of O
and of the gradients, so the results must be those of the original head dim -- checked against the CPU
oracle at that head dim, to the bars of the other parity tests (forward 2e-3 fp16 / 2e-2 bf16 absolute,
gradients 1e-2 / 3e-2 of their maximum).
"""
import numpy as np
import pytest
import torch

import oracle
from nvfuserexamples_amd import capi
from conftest import make_qkv, pad_mask, f32, rel_to_max

pytestmark = pytest.mark.gpu

TDT = {"fp16": torch.float16, "bf16": torch.bfloat16}
O_TOL = {"fp16": 2e-3, "bf16": 2e-2}
G_TOL = {"fp16": 1e-2, "bf16": 3e-2}

CASES = [
    # bh, sq, sk, d, dtype, causal, p_drop, masked
    (4, 128, 128, 32, "fp16", False, 0.0, False),
    (4, 200, 333, 96, "fp16", False, 0.1, True),    # ragged tiles, dropout, padding mask
    (4, 256, 256, 80, "bf16", True, 0.0, False),
    (2, 96, 160, 40, "fp16", True, 0.1, True),
    (3, 64, 64, 8, "fp16", False, 0.0, False),
    (2, 130, 70, 36, "fp16", False, 0.1, True),     # not a multiple of 8: padded to 40 by the operator
    (2, 200, 264, 256, "fp16", False, 0.1, True),   # head dim 256 itself (folded tensors)
    (2, 160, 160, 192, "bf16", True, 0.0, False),   # padded to 256
]


@pytest.mark.parametrize("bh,sq,sk,d,dtype,causal,p,masked", CASES)
def test_operators_take_other_head_dims(bh, sq, sk, d, dtype, causal, p, masked):
    from nvfuserexamples_amd import load_ops
    ops = load_ops()
    q, k, v, do = make_qkv(bh, sq, sk, d, seed=d + sq, dtype=dtype, with_dout=True)
    m = pad_mask(bh // 2 if bh % 2 == 0 else 1, sk, sk // 2, sk).to(TDT[dtype]) if masked else None
    mc = None if m is None else m.cuda()
    qc, kc, vc, doc = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    o, lse = ops.fmha_fwd(qc, kc, vc, mc, 0.0, causal, p, 9, 4)       # scale 0: 1/sqrt(d) of the ORIGINAL d
    dq, dk, dv = ops.fmha_bwd(doc, qc, kc, vc, o, lse, mc, 0.0, causal, p, 9, 4)
    torch.cuda.synchronize()
    assert o.shape == q.shape and o.is_contiguous() and lse.shape == (bh, sq)
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
    okw = dict(causal=causal)
    if p:
        okw.update(philox=True, p_drop=p, seed=9, offset=4)
    ref = oracle.attention(f32(q), f32(k), f32(v), mask=None if m is None else f32(m), dout=f32(do),
                           want=("o", "lse", "dq", "dk", "dv"), **okw)
    assert np.abs(f32(o.cpu()) - ref["o"]).max() <= O_TOL[dtype]
    assert np.abs(lse.cpu().numpy() - ref["lse"]).max() <= (2e-3 if dtype == "fp16" else 1e-2)
    for name, g in (("dq", dq), ("dk", dk), ("dv", dv)):
        assert rel_to_max(f32(g.cpu()), ref[name], floor=1e-3) <= G_TOL[dtype], name


NATIVE = [
    # bh, sq, sk, d, dtype, causal, p_drop, masked
    (4, 200, 333, 96, "fp16", False, 0.1, True),
    (4, 256, 320, 32, "bf16", True, 0.0, False),
    (2, 300, 300, 40, "fp16", True, 0.1, True),
    (2, 520, 520, 80, "fp16", False, 0.0, False),    # more than 256 rows: the two-kernel backward
    (2, 160, 264, 192, "bf16", False, 0.1, True),    # runs on the head-dim-256 kernels
    (2, 100, 100, 136, "fp16", True, 0.0, False),
    (3, 64, 64, 8, "fp16", False, 0.0, False),
]


@pytest.mark.parametrize("bh,sq,sk,d,dtype,causal,p,masked", NATIVE)
def test_c_abi_takes_head_dims_between_the_built_ones(bh, sq, sk, d, dtype, causal, p, masked):
    """Straight through the C ABI (which cannot pad: it allocates nothing), folded [bh, s, d] tensors."""
    q, k, v, do = make_qkv(bh, sq, sk, d, seed=3 * d + sq, dtype=dtype, with_dout=True)
    m = pad_mask(bh // 2, sk, sk // 2, sk).to(TDT[dtype]) if masked else None
    kw, okw = dict(causal=causal, scale=d ** -0.5), dict(causal=causal)
    if masked:
        kw["mask"] = m.cuda()
    if p:
        kw.update(drop_kind=capi.DROP_PHILOX, p_drop=p, seed=9, offset=4)
        okw.update(philox=True, p_drop=p, seed=9, offset=4)
    qc, kc, vc, doc = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    o, lse, _, _ = capi.fwd(qc, kc, vc, want_lse=True, **kw)
    dq, dk, dv = capi.bwd(doc, qc, kc, vc, o, lse, **kw)
    torch.cuda.synchronize()
    ref = oracle.attention(f32(q), f32(k), f32(v), mask=None if m is None else f32(m), dout=f32(do),
                           want=("o", "lse", "dq", "dk", "dv"), **okw)
    assert np.abs(f32(o.cpu()) - ref["o"]).max() <= O_TOL[dtype]
    assert np.abs(lse.cpu().numpy() - ref["lse"]).max() <= (2e-3 if dtype == "fp16" else 1e-2)
    for name, g in (("dq", dq), ("dk", dk), ("dv", dv)):
        assert rel_to_max(f32(g.cpu()), ref[name], floor=1e-3) <= G_TOL[dtype], name


@pytest.mark.parametrize("d", [24, 96, 200])
def test_columns_a_row_does_not_have_are_neither_read_nor_written(d):
    """Inputs and outputs are windows [..., :d] of wider rows: the columns behind them hold NaN on the way
    in (reading them would poison the results) and a sentinel on the way out (it must survive)."""
    b, h, s, wide = 2, 2, 200, d + 8
    q, k, v, do = make_qkv(b * h, s, s, d, seed=d, with_dout=True)

    def window(x, fill):
        buf = torch.full((b, s, h, wide), fill, dtype=torch.float16, device="cuda")
        win = buf[..., :d].permute(0, 2, 1, 3)
        if x is not None:
            win.copy_(x.view(b, h, s, d))
        return buf, win

    nan = float("nan")
    (_, q4), (_, k4), (_, v4), (_, do4) = (window(x, nan) for x in (q, k, v, do))
    obuf, o4 = window(None, 7.0)
    o4, lse, _, _ = capi.fwd(q4, k4, v4, want_lse=True, causal=True, scale=d ** -0.5, out=o4)
    gb = [window(None, 7.0) for _ in range(3)]
    dq, dk, dv = capi.bwd(do4, q4, k4, v4, o4, lse, causal=True, scale=d ** -0.5, grads=tuple(w for _, w in gb))
    torch.cuda.synchronize()
    for buf in (obuf, *(bf for bf, _ in gb)):
        assert torch.all(buf[..., d:] == 7.0)
    ref = oracle.attention(f32(q), f32(k), f32(v), causal=True, dout=f32(do), want=("o", "dq", "dk", "dv"))
    assert np.abs(f32(o4.reshape(b * h, s, d).cpu()) - ref["o"]).max() <= 2e-3
    for name, g in (("dq", dq), ("dk", dk), ("dv", dv)):
        assert rel_to_max(f32(g.reshape(b * h, s, d).cpu()), ref[name], floor=1e-3) <= 1e-2, name


def test_autograd_and_strided_views_at_head_dim_96():
    from nvfuserexamples_amd.autograd import attention
    b, h, s, d = 2, 3, 160, 96
    q, k, v, do = (t.cuda() for t in make_qkv(b * h, s, s, d, seed=12, with_dout=True))
    packed = torch.empty(b, s, 3, h, d, dtype=torch.float16, device="cuda")
    for i, x in enumerate((q, k, v)):
        packed[:, :, i] = x.view(b, h, s, d).permute(0, 2, 1, 3)
    packed.requires_grad_(True)
    qa, ka, va = (packed[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    o = attention(qa, ka, va, is_causal=True)
    assert o.shape == (b, h, s, d)
    o.backward(do.view(b, h, s, d))
    ref = oracle.attention(f32(q.cpu()), f32(k.cpu()), f32(v.cpu()), causal=True, dout=f32(do.cpu()),
                           want=("o", "dq", "dk", "dv"))
    assert np.abs(f32(o.detach().reshape(b * h, s, d).cpu()) - ref["o"]).max() <= 2e-3
    for i, name in enumerate(("dq", "dk", "dv")):
        g = packed.grad[:, :, i].permute(0, 2, 1, 3).reshape(b * h, s, d)
        assert rel_to_max(f32(g.cpu()), ref[name], floor=1e-3) <= 1e-2, name


def test_head_dims_beyond_the_built_ones_are_refused():
    """Beyond 256, and rows that are not whole 16-byte pieces at the C ABI: an error, never a wrong answer."""
    from nvfuserexamples_amd import load_ops
    ops = load_ops()
    x = torch.zeros(2, 64, 264, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        ops.fmha_fwd(x, x, x, None, 0.0, False, 0.0, 0, 0)
    w = torch.zeros(2, 64, 2, 264, dtype=torch.float16, device="cuda").transpose(1, 2)  # [B,H,S,D] view of [B,S,H,D]
    with pytest.raises(capi.FmhaError):
        capi.fwd(w, w, w)
    y = torch.zeros(2, 64, 36, dtype=torch.float16, device="cuda")
    with pytest.raises(capi.FmhaError):
        capi.fwd(y, y, y)
