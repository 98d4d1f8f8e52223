"""GPU parity of the backward path (dQ, dK, dV) through the C ABI.

Bar: max |g - oracle| / max |oracle| <= 1e-2 for fp16 (3e-2 for bf16), against the oracle's
analytic backward (itself pinned by finite differences and autograd in test_oracle.py).  The
forward that feeds the backward (O, LSE) is the library's own, as in a real train step."""
import numpy as np
import pytest
import torch

import oracle
from nvfuserexamples_amd import capi
from conftest import make_qkv, pad_mask, tail_mask, f32, rel_to_max

pytestmark = pytest.mark.gpu

TOL = {"fp16": 1e-2, "bf16": 3e-2}
TDT = {"fp16": torch.float16, "bf16": torch.bfloat16}

CASES = [
    # bh, sq, sk, d, dtype, mask, causal, p_drop
    (4, 128, 128, 64, "fp16", None, False, 0.0),
    (4, 128, 128, 64, "fp16", "pad", False, 0.0),
    (4, 128, 128, 64, "fp16", "add_full", False, 0.0),
    (4, 512, 512, 64, "fp16", "pad", False, 0.1),      # headline train-step shape (few heads)
    (3, 100, 77, 64, "fp16", None, False, 0.1),        # ragged
    (2, 70, 200, 64, "fp16", "add_full", False, 0.2),  # ragged + full mask + dropout
    (2, 1, 1, 64, "fp16", None, False, 0.0),
    (2, 320, 320, 64, "fp16", None, True, 0.0),        # causal
    (2, 200, 200, 64, "fp16", "pad", True, 0.1),       # causal + padding + dropout
    (2, 2048, 2048, 64, "fp16", None, False, 0.1),     # long sequence
    (2, 256, 256, 128, "fp16", None, False, 0.1),
    (2, 1024, 1024, 128, "bf16", None, True, 0.0),     # wide-head bf16 causal
    (4, 192, 192, 64, "bf16", "pad", False, 0.1),
    (4, 1, 1000, 64, "fp16", None, False, 0.0),        # one query against a long key range (decode step)
    (4, 300, 1, 64, "fp16", None, False, 0.0),         # one key: P = 1, dQ = dK = 0 exactly (with dropout the
                                                       # rounding of O in delta leaves ~3e-3 absolute in a zero gradient)
    (2, 130, 257, 64, "fp16", "add_full", False, 0.0), # full mask rows that are not 8-byte aligned
    (2, 192, 320, 128, "bf16", "add_full", False, 0.1),  # full mask tensor at head dim 128
    (2, 260, 260, 64, "bf16", "add_full", True, 0.1),  # full mask + causal + dropout
    (300, 128, 192, 64, "fp16", "add_full", False, 0.0),  # full mask, many workgroups
    # causal: a workgroup takes a pair of tiles (i, n-1-i); odd tile counts leave the middle one alone,
    # and with sk > sq the last key tiles see no query at all
    (3, 300, 300, 64, "fp16", None, True, 0.0),
    (2, 200, 333, 64, "fp16", None, True, 0.1),
    (2, 333, 200, 64, "fp16", "pad", True, 0.0),
    (2, 640, 640, 128, "bf16", None, True, 0.0),
    # head dim 256 (built for coverage, not tuned)
    (2, 256, 256, 256, "fp16", None, False, 0.0),
    (2, 200, 333, 256, "fp16", "pad", False, 0.1),
    (2, 130, 257, 256, "fp16", "add_full", False, 0.1),
    (2, 320, 320, 256, "bf16", None, True, 0.0),
    (3, 100, 77, 256, "bf16", "pad", True, 0.1),
    (2, 192, 192, 256, "fp16", "pad", True, 0.1),
]


@pytest.mark.parametrize("bh,sq,sk,d,dtype,mask,causal,p", CASES)
def test_backward_matches_oracle(bh, sq, sk, d, dtype, mask, causal, p):
    std = {64: 1.0, 128: 0.5, 256: 0.35}[d]
    q, k, v, do = make_qkv(bh, sq, sk, d, seed=bh + sk, std=std, dtype=dtype, with_dout=True)
    m = None
    if mask == "pad":
        m = pad_mask(bh // 2, sk, sk // 2, sk)
    elif mask == "add_full":
        m = torch.randn(bh, sq, sk, generator=torch.Generator().manual_seed(sq)) * 2
    if m is not None:
        m = m.to(TDT[dtype])
    kw = dict(causal=causal)
    okw = dict(causal=causal)
    if p > 0:
        kw.update(drop_kind=capi.DROP_PHILOX, p_drop=p, seed=99, offset=12)
        okw.update(philox=True, p_drop=p, seed=99, offset=12)
    qc, kc, vc, mc = q.cuda(), k.cuda(), v.cuda(), (None if m is None else m.cuda())
    o, lse, _, _ = capi.fwd(qc, kc, vc, mask=mc, want_lse=True, **kw)
    dq, dk, dv = capi.bwd(do.cuda(), qc, kc, vc, o, lse, mask=mc, **kw)
    torch.cuda.synchronize()
    ref = oracle.attention(f32(q), f32(k), f32(v), mask=None if m is None else f32(m), dout=f32(do),
                           want=("dq", "dk", "dv"), **okw)
    for name, t in (("dq", dq), ("dk", dk), ("dv", dv)):
        assert rel_to_max(f32(t.cpu()), ref[name], floor=1e-3) <= TOL[dtype], name


def test_backward_golden_fixture():
    import os
    f = np.load(os.path.join(os.path.dirname(__file__), "golden", "fwd_small.npz"))
    q, k, v, do, m = (torch.from_numpy(f[n]).half().cuda() for n in ("q", "k", "v", "dout", "mask"))
    kw = dict(drop_kind=capi.DROP_PHILOX, p_drop=float(f["p_drop"]), seed=int(f["seed"]), offset=int(f["offset"]))
    o, lse, _, _ = capi.fwd(q, k, v, mask=m, want_lse=True, **kw)
    dq, dk, dv = capi.bwd(do, q, k, v, o, lse, mask=m, **kw)
    for name, t in (("dq", dq), ("dk", dk), ("dv", dv)):
        assert rel_to_max(f32(t.cpu()), f[name]) <= 1e-2, name


def test_backward_properties_at_headline_shape():
    """B32 H16 S512 D64 train step: size-independent checks plus oracle parity on sampled heads."""
    B, H, S, D = 32, 16, 512, 64
    q, k, v, do = make_qkv(B * H, S, S, D, seed=0, with_dout=True)
    m = pad_mask(B, S, S // 2, S).half()
    kw = dict(drop_kind=capi.DROP_PHILOX, p_drop=0.1, seed=0x1234, offset=0)
    qc, kc, vc, dc, mc = q.cuda(), k.cuda(), v.cuda(), do.cuda(), m.cuda()
    o, lse, _, _ = capi.fwd(qc, kc, vc, mask=mc, want_lse=True, **kw)
    dq, dk, dv = capi.bwd(dc, qc, kc, vc, o, lse, mask=mc, **kw)
    # gradients are linear in dO
    dq2, dk2, dv2 = capi.bwd((dc.float() * 2).half(), qc, kc, vc, o, lse, mask=mc, **kw)
    for a, b in ((dq, dq2), (dk, dk2), (dv, dv2)):
        assert (b.float() - 2 * a.float()).abs().max().item() <= 1e-2 * b.float().abs().max().item()
        # (not bit for bit: many dS elements are fp16 subnormals, whose rounding does not commute with a doubling)
    # padded keys receive no gradient
    lens = (m[:, 0, 0] == 0).sum(-1)
    dkv = dk.view(B, H, S, D).float().abs() + dv.view(B, H, S, D).float().abs()
    for b in range(B):
        assert dkv[b, :, lens[b]:].max().item() == 0.0
    # sum_q dQ.Q == sum_k dK.K (softmax scores are bilinear in q and k)
    lhs = (dq.float() * qc.float()).sum((1, 2))
    rhs = (dk.float() * kc.float()).sum((1, 2))
    assert (lhs - rhs).abs().max().item() <= 2e-2 * lhs.abs().max().item()
    torch.cuda.synchronize()
    # oracle parity, dropout included, on sampled heads of the full batch: the oracle takes a head's
    # index in the whole problem (its Philox blocks are numbered by absolute head)
    for hd in (0, 100, 511):
        ref = oracle.attention(f32(q[hd:hd + 1]), f32(k[hd:hd + 1]), f32(v[hd:hd + 1]), dout=f32(do[hd:hd + 1]),
                               mask=f32(m[hd // H]).reshape(1, 1, S), want=("o", "dq", "dk", "dv"),
                               philox=True, p_drop=0.1, seed=0x1234, offset=0, bh_offset=hd)
        assert np.abs(f32(o[hd:hd + 1].cpu()) - ref["o"]).max() <= 2e-3
        for name, t in (("dq", dq), ("dk", dk), ("dv", dv)):
            assert rel_to_max(f32(t[hd:hd + 1].cpu()), ref[name]) <= 1e-2, (name, hd)


@pytest.mark.parametrize("bh,sq,sk,d,dtype,p", [(6, 300, 300, 64, "fp16", 0.1), (4, 200, 333, 64, "fp16", 0.0),
                                                 (4, 640, 512, 128, "bf16", 0.0)])
def test_causal_tile_pairing_is_bit_identical(bh, sq, sk, d, dtype, p, monkeypatch):
    """With a causal mask and enough heads a workgroup of the backward kernels takes a pair of tiles
    (i, n-1-i) so that all workgroups carry equal work.  Which tiles share a workgroup must not change
    a single bit: the paired schedule (forced here, it is otherwise chosen only for large batches) is
    compared with the one-tile-per-workgroup schedule that the oracle tests above exercise."""
    q, k, v, do = make_qkv(bh, sq, sk, d, seed=5, std=0.5 if d == 128 else 1.0, dtype=dtype, with_dout=True)
    qc, kc, vc, doc = (t.cuda() for t in (q, k, v, do))
    kw = dict(causal=True)
    if p:
        kw.update(drop_kind=capi.DROP_PHILOX, p_drop=p, seed=7, offset=3)
    o, lse, _, _ = capi.fwd(qc, kc, vc, want_lse=True, **kw)
    outs = []
    for pair in ("0", "1"):
        monkeypatch.setenv("FMHA_BWD_PAIR", pair)
        outs.append([t.clone() for t in capi.bwd(doc, qc, kc, vc, o, lse, **kw)])
        torch.cuda.synchronize()
    for a, b in zip(*outs):
        assert torch.equal(a, b)


FULL_SIZE = [
    # B, H, S, D, dtype, causal, p_drop, std          (the other train configurations, at full size)
    (4, 16, 2048, 64, "fp16", False, 0.1, 1.0),       # long sequences, Philox dropout, no mask
    (16, 32, 1024, 128, "bf16", True, 0.0, 0.5),      # wide heads, bf16, causal
]


@pytest.mark.parametrize("B,H,S,D,dtype,causal,p,std", FULL_SIZE)
def test_train_step_properties_at_full_size(B, H, S, D, dtype, causal, p, std):
    """Size-independent checks of forward + backward at the full size of the long-sequence and the
    wide-head configuration, plus oracle parity on the first two heads (the oracle draws its keep
    decisions by absolute head index, so heads 0 and 1 of the batch are heads 0 and 1 there)."""
    bh = B * H
    tdt = TDT[dtype]
    q, k, v, do = make_qkv(bh, S, S, D, seed=3, std=std, dtype=dtype, with_dout=True)
    kw = dict(causal=causal)
    okw = dict(causal=causal)
    if p:
        kw.update(drop_kind=capi.DROP_PHILOX, p_drop=p, seed=0x1234, offset=0)
        okw.update(philox=True, p_drop=p, seed=0x1234, offset=0)
    qc, kc, vc, dc = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    o, lse, _, _ = capi.fwd(qc, kc, vc, want_lse=True, **kw)
    dq, dk, dv = capi.bwd(dc, qc, kc, vc, o, lse, **kw)
    gtol = 1e-2 if dtype == "fp16" else 3e-2
    # gradients are linear in dO (doubling is exact in both element types)
    g2 = capi.bwd((dc.float() * 2).to(tdt), qc, kc, vc, o, lse, **kw)
    for a, b in zip((dq, dk, dv), g2):
        assert (b.float() - 2 * a.float()).abs().max().item() <= gtol * b.float().abs().max().item()
    # sum_q dQ.Q == sum_k dK.K per head (the scores are bilinear in q and k)
    lhs = (dq.float() * qc.float()).sum((1, 2))
    rhs = (dk.float() * kc.float()).sum((1, 2))
    assert (lhs - rhs).abs().max().item() <= 2 * gtol * lhs.abs().max().item()
    if causal:
        # the future does not reach the past: new K, V rows at the end leave earlier queries' O bit for bit
        cut = S - 100
        k2, v2 = kc.clone(), vc.clone()
        k2[:, cut:] = 1.0
        v2[:, cut:] = -3.0
        o2 = capi.fwd(qc, k2, v2, **kw)[0]
        assert torch.equal(o2[:, :cut], o[:, :cut])
        assert not torch.equal(o2[:, cut:], o[:, cut:])
    torch.cuda.synchronize()
    heads = [0, 1]
    ref = oracle.attention(f32(q[heads]), f32(k[heads]), f32(v[heads]), dout=f32(do[heads]),
                           want=("o", "dq", "dk", "dv"), **okw)
    assert np.abs(f32(o[heads].cpu()) - ref["o"]).max() <= (2e-3 if dtype == "fp16" else 2e-2)
    for name, t in zip(("dq", "dk", "dv"), (dq, dk, dv)):
        assert rel_to_max(f32(t[heads].cpu()), ref[name]) <= gtol, name


# Heads of at most 256 queries and 256 keys (head dim 64, no full mask tensor) take one launch:
# the workgroup copies Q, K, V and dO into LDS once and computes dQ, then dK and dV, from that copy.
# FMHA_BWD_SHORT=0 keeps the same calls on the two general kernels; both must meet the oracle.
SHORT_SEQ = [
    # bh, sq, sk, dtype, mask, p_drop, kv_len, causal
    (4, 128, 128, "fp16", None, 0.0, False, False),
    (6, 128, 128, "fp16", "pad", 0.1, False, False),       # BERT-base train step shape (few heads)
    (3, 100, 77, "fp16", None, 0.1, False, False),         # ragged in both directions
    (5, 33, 128, "bf16", "pad", 0.1, False, False),        # queries fill one wave and a bit
    (4, 128, 40, "fp16", "pad", 0.0, False, False),        # keys fill one wave and a bit: two waves idle in the second phase
    (4, 64, 64, "fp16", "inf", 0.2, False, False),         # one LDS tile per matrix; -inf mask entries
    (2, 1, 1, "fp16", None, 0.0, False, False),
    (600, 128, 128, "fp16", "pad", 0.1, False, False),     # more workgroups than the device holds at once
    (8, 96, 128, "fp16", None, 0.1, True, False),          # valid key counts
    # up to 256 rows: the same kernel with eight waves and 128 KB of LDS
    (4, 256, 256, "fp16", "pad", 0.1, False, False),
    (6, 197, 197, "fp16", None, 0.1, False, False),        # ViT-B/16 sequence length
    (3, 130, 250, "bf16", "pad", 0.0, False, False),       # five query blocks against eight key blocks
    (300, 200, 250, "fp16", "pad", 0.1, False, False),     # more workgroups than the device holds at once
    (8, 256, 200, "fp16", None, 0.0, True, False),         # valid key counts
    # causal (key <= query): blocks above the diagonal are skipped in both phases
    (4, 128, 128, "fp16", None, 0.0, False, True),
    (6, 200, 200, "fp16", "pad", 0.1, False, True),
    (3, 77, 250, "bf16", None, 0.1, False, True),   # more keys than queries: the last key blocks see no query
    (3, 250, 100, "fp16", None, 0.0, False, True),  # more queries than keys
    (8, 256, 256, "fp16", None, 0.1, True, True),   # causal with valid key counts
]


@pytest.mark.parametrize("short", ["1", "0"])
@pytest.mark.parametrize("bh,sq,sk,dtype,mask,p,use_len,causal", SHORT_SEQ)
def test_short_sequences_backward(bh, sq, sk, dtype, mask, p, use_len, causal, short, monkeypatch):
    monkeypatch.setenv("FMHA_BWD_SHORT", short)
    q, k, v, do = make_qkv(bh, sq, sk, 64, seed=bh + sk, dtype=dtype, with_dout=True)
    m = None
    if mask == "pad":
        m = pad_mask(bh // 2 if bh % 2 == 0 else 1, sk, max(1, sk // 2), sk)
    elif mask == "inf":
        m = torch.randn(bh, 1, sk, generator=torch.Generator().manual_seed(sk)) * 2
        m[:, :, 3::5] = float("-inf")
    if m is not None:
        m = m.to(TDT[dtype])
    kw, okw = dict(causal=causal), dict(causal=causal)
    if p > 0:
        kw.update(drop_kind=capi.DROP_PHILOX, p_drop=p, seed=99, offset=12)
        okw.update(philox=True, p_drop=p, seed=99, offset=12)
    mo = None if m is None else f32(m)
    if use_len:
        lens = torch.tensor([sk, 1, 5, sk // 2], dtype=torch.int32)
        kw["kv_len"] = lens.cuda()
        mo = np.zeros((4, 1, 1, sk), np.float32)
        for i, n in enumerate(lens.tolist()):
            mo[i, 0, 0, n:] = -np.inf
    qc, kc, vc, mc = q.cuda(), k.cuda(), v.cuda(), (None if m is None else m.cuda())
    o, lse, _, _ = capi.fwd(qc, kc, vc, mask=mc, want_lse=True, **kw)
    dq, dk, dv = capi.bwd(do.cuda(), qc, kc, vc, o, lse, mask=mc, **kw)
    torch.cuda.synchronize()
    ref = oracle.attention(f32(q), f32(k), f32(v), mask=mo, dout=f32(do), want=("dq", "dk", "dv"), **okw)
    for name, t in (("dq", dq), ("dk", dk), ("dv", dv)):
        got = f32(t.cpu())
        assert np.isfinite(got).all(), name
        assert rel_to_max(got, ref[name], floor=1e-3) <= TOL[dtype], name
    if use_len:
        # keys past a sequence's count get no gradient at all, and a sequence without keys none anywhere
        per = bh // 4
        for i, n in enumerate(lens.tolist()):
            sl = slice(i * per, (i + 1) * per)
            assert not dk[sl, n:].any() and not dv[sl, n:].any()
        # a sequence without any key: O = 0, LSE = -inf, and no gradient anywhere (nothing non-finite either)
        lens[1] = 0
        kw["kv_len"] = lens.cuda()
        o, lse, _, _ = capi.fwd(qc, kc, vc, want_lse=True, **kw)
        g0 = capi.bwd(do.cuda(), qc, kc, vc, o, lse, **kw)
        torch.cuda.synchronize()
        sl = slice(per, 2 * per)
        for t in g0:
            assert torch.isfinite(t.float()).all() and not t[sl].any()


@pytest.mark.parametrize("bh,sq,sk,mask,p,std", [
    (4, 512, 512, "pad", 0.0, 3.0),      # pipelined forward (lazily re-based softmax), general backward
    (4, 128, 128, "add_full", 0.0, 3.0), # one-pass short-range forward
    (4, 300, 520, "add_full", 0.0, 6.0), # streaming forward: |LSE| up to ~190
    (4, 256, 256, None, 0.1, 4.0),       # one-launch backward
])
def test_large_scores_stay_finite_and_accurate(bh, sq, sk, mask, p, std):
    """Scores far outside the usual range (|LSE| 40-190 instead of ~6): nothing overflows, and the
    errors stay proportional to the size of the scores (the pipelined kernels round Q * scale once to
    the element type, so each score carries 2^-11 of its own magnitude)."""
    q, k, v, do = make_qkv(bh, sq, sk, 64, seed=sq + sk, std=std, with_dout=True)
    v, do = (v / std).half(), (do / std).half()
    m = None
    if mask == "pad":
        m = pad_mask(bh // 2, sk, sk // 2, sk).half()
    elif mask == "add_full":
        m = (torch.randn(bh, sq, sk, generator=torch.Generator().manual_seed(sq)) * 3).half()
    kw, okw = {}, {}
    if p:
        kw.update(drop_kind=capi.DROP_PHILOX, p_drop=p, seed=1, offset=2)
        okw.update(philox=True, p_drop=p, seed=1, offset=2)
    mc = None if m is None else m.cuda()
    o, lse, _, _ = capi.fwd(q.cuda(), k.cuda(), v.cuda(), mask=mc, want_lse=True, **kw)
    dq, dk, dv = capi.bwd(do.cuda(), q.cuda(), k.cuda(), v.cuda(), o, lse, mask=mc, **kw)
    torch.cuda.synchronize()
    ref = oracle.attention(f32(q), f32(k), f32(v), mask=None if m is None else f32(m), dout=f32(do),
                           want=("o", "lse", "dq", "dk", "dv"), **okw)
    assert np.abs(ref["lse"]).max() > 30
    assert np.abs(f32(o.cpu()) - ref["o"]).max() <= 2e-2
    assert np.abs(lse.cpu().numpy() - ref["lse"]).max() <= 1e-3 * np.abs(ref["lse"]).max()
    for name, t in (("dq", dq), ("dk", dk), ("dv", dv)):
        got = f32(t.cpu())
        assert np.isfinite(got).all(), name
        assert rel_to_max(got, ref[name]) <= 3e-2, name


@pytest.mark.parametrize("bh,s,d,dtype", [(8, 8192, 64, "fp16"), (4, 4096, 128, "bf16")])
def test_long_sequences_split_over_keys(bh, s, d, dtype):
    """Sequences far beyond what the oracle finishes in seconds (128 key tiles), checked by an identity
    instead: attention over all keys is the LSE-weighted merge of attention over the two halves of the
    keys, and, given the full O and LSE, the backward over half the keys yields that half's dK and dV
    and a dQ that sums to the full one."""
    tdt = TDT[dtype]
    q, k, v, do = (t.cuda() for t in make_qkv(bh, s, s, d, seed=s, std=0.5 if d == 128 else 1.0, dtype=dtype,
                                              with_dout=True))
    o, lse, _, _ = capi.fwd(q, k, v, want_lse=True)
    h = s // 2
    halves = [(k[:, :h].contiguous(), v[:, :h].contiguous()), (k[:, h:].contiguous(), v[:, h:].contiguous())]
    parts = [capi.fwd(q, kk, vv, want_lse=True)[:2] for kk, vv in halves]
    l1, l2 = parts[0][1].double(), parts[1][1].double()
    lm = torch.logaddexp(l1, l2)
    merged = parts[0][0].double() * (l1 - lm).exp().unsqueeze(-1) + parts[1][0].double() * (l2 - lm).exp().unsqueeze(-1)
    otol = 2e-3 if dtype == "fp16" else 2e-2
    assert (merged - o.double()).abs().max().item() <= otol
    assert (lm - lse.double()).abs().max().item() <= 2e-3
    # backward: the same O and LSE, half of the keys at a time
    dq, dk, dv = capi.bwd(do, q, k, v, o, lse)
    g = [capi.bwd(do, q, kk, vv, o, lse) for kk, vv in halves]
    gtol = 1e-2 if dtype == "fp16" else 3e-2
    for full, a, b in ((dk, g[0][1], g[1][1]), (dv, g[0][2], g[1][2])):
        cat = torch.cat([a, b], dim=1).float()
        assert (cat - full.float()).abs().max().item() <= gtol * full.float().abs().max().item()
    dq_sum = g[0][0].float() + g[1][0].float()
    assert (dq_sum - dq.float()).abs().max().item() <= gtol * dq.float().abs().max().item()
    assert torch.isfinite(dq.float()).all() and torch.isfinite(dk.float()).all() and torch.isfinite(dv.float()).all()


# A [B,1,1,sk] mask that ends in hard-masked keys lets the dQ kernel stop at the last live key tile
# and the dK/dV kernel leave out key tiles past it.  Those keys have P = 0 exactly either way, so the
# gradients must equal, bit for bit, those of launches that visit every tile (FLAG_NO_MASK_TRIM).
BWD_TRIM = [
    # bh, sq, sk, d, dtype, kind, causal, p, kv_len
    (8, 512, 512, 64, "fp16", "tail", False, 0.0, False),
    (8, 512, 512, 64, "fp16", "tail", False, 0.1, False),     # headline train-step shape (few heads)
    (8, 512, 512, 64, "fp16", "inf", False, 0.0, False),
    (8, 512, 512, 64, "fp16", "holes", False, 0.1, False),
    (8, 512, 512, 64, "fp16", "soft", False, 0.0, False),
    (8, 300, 512, 64, "fp16", "last_live", False, 0.0, False),
    (8, 512, 512, 64, "fp16", "some_rows_all_masked", False, 0.1, False),
    (6, 300, 333, 64, "bf16", "tail", False, 0.1, False),
    (4, 300, 1024, 64, "fp16", "tail", False, 0.0, False),    # the longest rows that are looked at
    (4, 300, 1100, 64, "fp16", "tail", False, 0.0, False),    # beyond: not looked at
    (4, 320, 320, 128, "bf16", "tail", False, 0.1, False),
    (2, 300, 333, 256, "fp16", "holes", False, 0.1, False),   # head dim 256: 32-row tiles
    (4, 384, 384, 64, "fp16", "tail", True, 0.1, False),      # causal: tile pairs, both limits apply
    (8, 512, 512, 64, "fp16", "holes", False, 0.0, True),     # valid key counts on top of the mask
]


@pytest.mark.parametrize("bh,sq,sk,d,dtype,kind,causal,p,use_len", BWD_TRIM)
def test_trailing_hard_masked_keys_are_skipped_exactly(bh, sq, sk, d, dtype, kind, causal, p, use_len):
    b = bh // 2
    q, k, v, do = make_qkv(bh, sq, sk, d, seed=bh + sk, std={64: 1.0, 128: 0.5, 256: 0.35}[d], dtype=dtype, with_dout=True)
    m = tail_mask(kind, b, sk, seed=sk + bh).to(TDT[dtype])
    kw = dict(mask=m.cuda(), causal=causal)
    okw = dict(causal=causal)
    if p > 0:
        kw.update(drop_kind=capi.DROP_PHILOX, p_drop=p, seed=5, offset=1)
        okw.update(philox=True, p_drop=p, seed=5, offset=1)
    if use_len:
        kv = torch.randint(0, sk + 1, (b,), generator=torch.Generator().manual_seed(5), dtype=torch.int32)
        kw.update(kv_len=kv.cuda())
    qc, kc, vc, doc = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    o, lse, _, _ = capi.fwd(qc, kc, vc, want_lse=True, **kw)
    grads = capi.bwd(doc, qc, kc, vc, o, lse, **kw)
    grads_all = capi.bwd(doc, qc, kc, vc, o, lse, flags=capi.FLAG_NO_MASK_TRIM, **kw)
    torch.cuda.synchronize()
    for name, t, t_all in zip(("dq", "dk", "dv"), grads, grads_all):
        assert torch.equal(t, t_all), name
    if not use_len:
        ref = oracle.attention(f32(q), f32(k), f32(v), mask=f32(m), dout=f32(do), want=("dq", "dk", "dv"), **okw)
        for name, t in zip(("dq", "dk", "dv"), grads):
            assert rel_to_max(f32(t.cpu()), ref[name], floor=1e-3) <= TOL[dtype], name


# Key ranges of 257 to 512 keys at head dim 64 (the shapes an earlier one-pass kernel served; kept as coverage of
# the two-kernel path: ragged tiles, one query, hard-masked tails, valid key counts).
MIDDLE_RANGES = [
    # bh, sq, sk, dtype, mask, p_drop
    (4, 512, 512, "fp16", "pad", 0.1),     # headline train-step shape (few heads): two key chunks
    (4, 512, 512, "fp16", None, 0.0),
    (3, 300, 300, "fp16", None, 0.1),      # ragged tiles and a partly filled second chunk
    (3, 100, 477, "fp16", "pad", 0.1),
    (2, 700, 260, "fp16", "pad", 0.0),     # four keys in the second chunk
    (2, 64, 512, "bf16", "pad", 0.1),
    (2, 333, 257, "bf16", None, 0.0),
    (5, 1, 300, "fp16", None, 0.0),        # one query
    (6, 512, 512, "fp16", "tail", 0.1),    # hard-masked tails of every length: chunks and key blocks left out
    (6, 384, 512, "fp16", "holes", 0.1),
    (4, 512, 512, "fp16", "kvlen", 0.1),   # valid key counts 100, 256, 257, 512
    (3, 320, 256, "fp16", "pad", 0.1),     # one chunk: no workspace involved
]


@pytest.mark.parametrize("bh,sq,sk,dtype,mask,p", MIDDLE_RANGES)
def test_backward_of_middle_key_ranges_matches_oracle(bh, sq, sk, dtype, mask, p):
    q, k, v, do = make_qkv(bh, sq, sk, 64, seed=bh + sk, dtype=dtype, with_dout=True)
    m = kvl = None
    if mask == "pad":
        m = pad_mask(bh // 2 if bh % 2 == 0 else bh, sk, sk // 2, sk)
    elif mask in ("tail", "holes"):
        m = tail_mask(mask, bh, sk, 5)
    elif mask == "kvlen":
        kvl = torch.tensor([100, 256, 257, 512][:bh], dtype=torch.int32)
    if m is not None:
        m = m.to(TDT[dtype])
    kw, okw = {}, {}
    if p > 0:
        kw.update(drop_kind=capi.DROP_PHILOX, p_drop=p, seed=99, offset=12)
        okw.update(philox=True, p_drop=p, seed=99, offset=12)
    qc, kc, vc, mc = q.cuda(), k.cuda(), v.cuda(), (None if m is None else m.cuda())
    kvc = None if kvl is None else kvl.cuda()
    o, lse, _, _ = capi.fwd(qc, kc, vc, mask=mc, want_lse=True, kv_len=kvc, **kw)
    dq, dk, dv = capi.bwd(do.cuda(), qc, kc, vc, o, lse, mask=mc, kv_len=kvc, **kw)
    torch.cuda.synchronize()
    om = None if m is None else f32(m)
    if kvl is not None:
        om = np.zeros((bh, 1, sk), np.float32)
        for i in range(bh):
            om[i, 0, int(kvl[i]):] = -np.inf
    ref = oracle.attention(f32(q), f32(k), f32(v), mask=om, dout=f32(do), want=("dq", "dk", "dv"), **okw)
    for name, t in zip(("dq", "dk", "dv"), (dq, dk, dv)):
        assert rel_to_max(f32(t.cpu()), ref[name], floor=1e-3) <= TOL[dtype], name


def test_flag_of_the_removed_one_pass_kernel_is_accepted_and_ignored():
    """flags bit 2 asked for a one-pass kernel in earlier versions of the C ABI; it changes nothing now, and no
    backward asks for a workspace."""
    q, k, v, do = make_qkv(3, 300, 400, 64, seed=3, with_dout=True)
    qc, kc, vc, dc = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    o, lse, _, _ = capi.fwd(qc, kc, vc, want_lse=True)
    a = capi.bwd(dc, qc, kc, vc, o, lse, flags=2)
    b = capi.bwd(dc, qc, kc, vc, o, lse)
    for x, y in zip(a, b):
        assert torch.equal(x, y)
    assert capi.lib().fmha_bwd_workspace_bytes(3, 300, 400, 64) == 0
