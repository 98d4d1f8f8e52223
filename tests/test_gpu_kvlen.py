"""Valid key counts (`kv_len`): the "padded version" the reference leaves as a TODO
(reference fmha/fmha_manual.cpp:110,178).  Head b attends keys [0, kv_len[b / div]) only, exactly
as if the other keys carried a -inf mask; key tiles past the count are skipped by the kernels.

Checked against the CPU oracle fed with the equivalent -inf additive mask (same tolerances as the
other parity tests), and bit for bit against this build's own additive -10000 padding-mask path,
whose masked probabilities underflow to exactly zero.
"""
import numpy as np
import pytest
import torch

import oracle
from nvfuserexamples_amd import capi
from conftest import make_qkv, f32, rel_to_max

pytestmark = pytest.mark.gpu

TDT = {"fp16": torch.float16, "bf16": torch.bfloat16}
O_TOL = {"fp16": 2e-3, "bf16": 2e-2}
G_TOL = {"fp16": 1e-2, "bf16": 3e-2}


def _lens(b, sk, seed, lo=1):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, sk + 1, (b,), generator=g, dtype=torch.int32)


def _inf_mask(lens, heads_per_len, sq, sk):
    """[bh,sq,sk] additive mask: -inf at keys >= the head's count."""
    b = lens.numel()
    m = torch.zeros(b, 1, sk)
    for i, n in enumerate(lens.tolist()):
        m[i, 0, n:] = float("-inf")
    return m.repeat_interleave(heads_per_len, 0).expand(b * heads_per_len, sq, sk).contiguous()


CASES = [
    # bh, groups, sq, sk, d, dtype, causal, p_drop
    (8, 4, 128, 128, 64, "fp16", False, 0.0),
    (6, 3, 200, 333, 64, "fp16", False, 0.1),     # ragged, dropout
    (6, 6, 320, 320, 64, "fp16", True, 0.0),      # causal
    (4, 2, 256, 256, 128, "bf16", False, 0.0),
    (600, 300, 128, 192, 64, "fp16", False, 0.0),  # more items than resident workgroups: per-item counts
    (4, 2, 200, 333, 256, "fp16", False, 0.1),     # head dim 256: the plain forward loop reads the counts too
    (4, 4, 192, 192, 256, "bf16", True, 0.0),
]


@pytest.mark.parametrize("bh,b,sq,sk,d,dtype,causal,p", CASES)
def test_kv_len_matches_oracle_with_inf_mask(bh, b, sq, sk, d, dtype, causal, p):
    q, k, v, do = make_qkv(bh, sq, sk, d, seed=bh + sk, std={64: 1.0, 128: 0.5, 256: 0.35}[d], dtype=dtype, with_dout=True)
    lens = _lens(b, sk, seed=sk)
    kw, okw = dict(causal=causal), dict(causal=causal)
    if p:
        kw.update(drop_kind=capi.DROP_PHILOX, p_drop=p, seed=11, offset=5)
        okw.update(philox=True, p_drop=p, seed=11, offset=5)
    qc, kc, vc, doc, lc = q.cuda(), k.cuda(), v.cuda(), do.cuda(), lens.cuda()
    o, lse, _, _ = capi.fwd(qc, kc, vc, kv_len=lc, want_lse=True, **kw)
    dq, dk, dv = capi.bwd(doc, qc, kc, vc, o, lse, kv_len=lc, **kw)
    torch.cuda.synchronize()
    m = _inf_mask(lens, bh // b, sq, sk)
    ref = oracle.attention(f32(q), f32(k), f32(v), mask=m.numpy(), dout=f32(do), want=("o", "lse", "dq", "dk", "dv"),
                           **okw)
    assert np.abs(f32(o.cpu()) - ref["o"]).max() <= O_TOL[dtype]
    for name, g in (("dq", dq), ("dk", dk), ("dv", dv)):
        assert rel_to_max(f32(g.cpu()), ref[name], floor=1e-3) <= G_TOL[dtype], name
    # keys past a head's count receive no gradient at all
    for i, n in enumerate(lens.tolist()):
        hs = slice(i * (bh // b), (i + 1) * (bh // b))
        assert not dk[hs, n:].any() and not dv[hs, n:].any()


@pytest.mark.parametrize("bh,b,s,d", [(32, 4, 512, 64), (8, 2, 384, 128)])
def test_kv_len_equals_additive_padding_mask_bit_for_bit(bh, b, s, d):
    q, k, v, do = make_qkv(bh, s, s, d, seed=3, std=0.5 if d == 128 else 1.0, with_dout=True)
    lens = _lens(b, s, seed=9, lo=s // 2)
    pad = torch.zeros(b, 1, 1, s)
    for i, n in enumerate(lens.tolist()):
        pad[i, ..., n:] = -10000.0
    qc, kc, vc, doc = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    o1, l1, _, _ = capi.fwd(qc, kc, vc, kv_len=lens.cuda(), want_lse=True)
    o2, l2, _, _ = capi.fwd(qc, kc, vc, mask=pad.half().cuda(), want_lse=True)
    assert torch.equal(o1, o2) and torch.equal(l1, l2)
    g1 = capi.bwd(doc, qc, kc, vc, o1, l1, kv_len=lens.cuda())
    g2 = capi.bwd(doc, qc, kc, vc, o2, l2, mask=pad.half().cuda())
    torch.cuda.synchronize()
    for a, c in zip(g1, g2):
        assert torch.equal(a, c)


@pytest.mark.parametrize("d", [64, 256])
def test_zero_count_gives_zero_output(d):
    q, k, v = make_qkv(4, 64, 96, d, seed=1, std=0.5)
    lens = torch.tensor([0, 40], dtype=torch.int32)
    o, lse, _, _ = capi.fwd(q.cuda(), k.cuda(), v.cuda(), kv_len=lens.cuda(), want_lse=True)
    torch.cuda.synchronize()
    assert not o[:2].any() and torch.isinf(lse[:2]).all() and (lse[:2] < 0).all()
    assert torch.isfinite(lse[2:]).all()


def test_kv_len_through_the_operator_and_autograd():
    from nvfuserexamples_amd import load_ops
    from nvfuserexamples_amd.autograd import attention
    ops = load_ops()
    q, k, v, do = make_qkv(8, 128, 160, 64, seed=2, with_dout=True)
    lens = _lens(4, 160, seed=4).cuda()
    qc, kc, vc = (t.cuda().requires_grad_() for t in (q, k, v))
    out = attention(qc, kc, vc, kv_len=lens)
    out.backward(do.cuda())
    o, lse = ops.fmha_fwd(q.cuda(), k.cuda(), v.cuda(), None, 0.0, False, 0.0, 0, 0, lens)
    assert torch.equal(out.detach(), o)
    dq, dk, dv = capi.bwd(do.cuda(), q.cuda(), k.cuda(), v.cuda(), o, lse, kv_len=lens)
    assert torch.equal(qc.grad, dq) and torch.equal(kc.grad, dk) and torch.equal(vc.grad, dv)
