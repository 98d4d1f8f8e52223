"""Head dims other than the two the kernels are built for (64 and 128).

The reference is fixed at D = 64 (fmha/fmha_manual.cpp:39-47).  The general operators accept any
head dim up to 128 by zero-padding to the next built size either side of the kernels: zero columns
change neither Q.K^T nor the kept columns of O and of the gradients, so the results must be those
of the original head dim -- checked against the CPU oracle at that head dim, to the bars of the
other parity tests (forward 2e-3 fp16 / 2e-2 bf16 absolute, gradients 1e-2 / 3e-2 of their maximum).
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
    (2, 200, 264, 256, "fp16", False, 0.1, True),   # head dim 256 itself (folded tensors)
    (2, 160, 160, 192, "bf16", True, 0.0, False),   # padded to 256
]


@pytest.mark.parametrize("bh,sq,sk,d,dtype,causal,p,masked", CASES)
def test_operators_pad_other_head_dims(bh, sq, sk, d, dtype, causal, p, masked):
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
    """Beyond 256: an error, never a wrong answer."""
    from nvfuserexamples_amd import load_ops
    ops = load_ops()
    x = torch.zeros(2, 64, 264, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        ops.fmha_fwd(x, x, x, None, 0.0, False, 0.0, 0, 0)
    w = torch.zeros(2, 64, 2, 264, dtype=torch.float16, device="cuda").transpose(1, 2)  # [B,H,S,D] view of [B,S,H,D]
    with pytest.raises(capi.FmhaError):
        capi.fwd(w, w, w)
