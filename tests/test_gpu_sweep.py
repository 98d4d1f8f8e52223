"""Seeded randomized parity sweep: forward and backward through the C ABI against the CPU oracle over
400 small problems that mix head dims (the built 64 / 128 / 256 and others between them), element types, ragged sizes, mask kinds (padding with -10000 or
-inf tails, holes, per-key, full tensors), causal masking, Philox dropout, valid key counts and strided
layouts.  Bars as everywhere else: |O - oracle| <= 2e-3 (fp16) / 2e-2 (bf16) (scaled up where |O|
exceeds 2), gradients within 1e-2 / 3e-2 of the largest oracle entry, LSE within 5e-3 + 2^-8 |LSE|,
-inf rows in the same places; where a per-key mask is involved, skipping the hard-masked tail must not
change a bit.

Gradients that are exactly zero.  When every query of a head sees exactly one key (sk = 1, a valid
length of 1, a causal first row alone), softmax is the constant 1 and dQ = dK = 0.  The kernels then
compute dS_i = P_i (dP_i - delta_i) with dP_i = Z (dO_i . V_k) and delta_i = dO_i . O_i, where O_i is the
forward's output ROUNDED to the element type: O_i = round(Z V_k).  The two terms differ by
dO_i . (Z V_k - round(Z V_k)), at most u * A_i with A_i = sum_d |dO_id O_id| and u the unit roundoff of
the element type (2^-11 fp16, 2^-8 bf16); without dropout Z = 1, round(V_k) = V_k and what is left is the
2^-2p relative error of the hi + lo split that carries delta and LSE into the matrix pipe, far below
that.  Hence |dQ_id| <= scale * u * A_i * |K_kd| and, the signs of the row errors being independent,
|dK_kd| is of the order scale * u * sqrt(sum_i A_i^2) * max|Q|.  Such all-zero gradients are judged on
ABSOLUTE error against 4 * scale * u * sqrt(sum_i A_i^2) * max(|Q|, |K|) instead of relative to a
maximum that does not exist."""
import os
import random

import numpy as np
import pytest
import torch

import oracle
from nvfuserexamples_amd import capi
from conftest import make_qkv, f32, rel_to_max

pytestmark = pytest.mark.gpu

TDT = {"fp16": torch.float16, "bf16": torch.bfloat16}
UNIT = {"fp16": 2.0 ** -11, "bf16": 2.0 ** -8}


def _case(it, rng, forced=None):
    c = forced or dict(
        d=rng.choice([64, 64, 64, 128, 256, 64, 128, 32, 96, 40, 200, 8]), dtype=rng.choice(["fp16", "fp16", "bf16"]),
        b=rng.choice([1, 2, 3]), h=rng.choice([1, 2, 4]),
        sq=rng.choice([1, 7, 31, 32, 33, 64, 65, 100, 127, 128, 129, 191, 200, 255, 256, 257, 300, 384, 520]),
        sk=rng.choice([1, 5, 8, 31, 32, 33, 40, 64, 65, 96, 127, 128, 129, 192, 200, 250, 256, 257, 300, 333, 512, 700]),
        causal=rng.random() < 0.3, p=rng.choice([0.0, 0.0, 0.1, 0.3]),
        mask=rng.choice(["none", "pad", "pad", "pad", "full", "keyinf", "padinf", "padholes"]),
        want_len=rng.random() < 0.3, want_strided=rng.random() < 0.25,
        spare=rng.random())  # (a draw an earlier option used: kept so that the sequence of cases stays the same)
    c.setdefault("lens", None)
    c["use_len"] = c["mask"] == "none" and c.get("want_len", False)
    c["strided"] = c.get("want_strided", False) and c["mask"] != "full"
    if c["d"] > 128 and c["sq"] * c["sk"] > 300 * 300:   # keep the CPU oracle's share of the minute small
        c["sq"], c["sk"] = min(c["sq"], 200), min(c["sk"], 257)
    return c


def _run_case(it, c, rng):
    d, dtype, b, h, sq, sk, causal, p, maskk = (c[n] for n in ("d", "dtype", "b", "h", "sq", "sk", "causal", "p", "mask"))
    bh = b * h
    std = 1.0 if d <= 64 else 0.5 if d <= 128 else 0.35
    q, k, v, do = make_qkv(bh, sq, sk, d, seed=it, std=std, dtype=dtype, with_dout=True)
    g = torch.Generator().manual_seed(it)
    m = mo = None
    if maskk in ("pad", "padinf", "padholes"):
        m = torch.zeros(b, 1, 1, sk)
        lens = c["lens"] or [rng.randint(1, sk) for _ in range(b)]
        for i in range(b):
            m[i, 0, 0, lens[i]:] = -10000.0 if maskk != "padinf" else float("-inf")
        if maskk == "padholes":
            m[:, :, :, torch.rand(sk, generator=g) < 0.3] = -10000.0
    elif maskk == "full":
        m = torch.randn(bh, sq, sk, generator=g) * 2
    elif maskk == "keyinf":
        m = torch.randn(bh, 1, sk, generator=g)
        m[:, :, 1::3] = float("-inf")
    if m is not None:
        m = m.to(TDT[dtype])
        mo = f32(m)
    kw, okw = dict(causal=causal), dict(causal=causal)
    if p:
        kw.update(drop_kind=capi.DROP_PHILOX, p_drop=p, seed=it * 7 + 1, offset=it)
        okw.update(philox=True, p_drop=p, seed=it * 7 + 1, offset=it)
    if c["use_len"]:
        lens = torch.tensor([rng.randint(1, sk) for _ in range(b)], dtype=torch.int32)
        kw["kv_len"] = lens.cuda()
        mo = np.zeros((b, 1, 1, sk), np.float32)
        for i, n in enumerate(lens.tolist()):
            mo[i, 0, 0, n:] = -np.inf
    qc, kc, vc, dc = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    if c["strided"]:
        def f(x):
            return x.view(b, h, x.shape[1], d).permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
        qc, kc, vc, dc = f(qc), f(kc), f(vc), f(dc)
    mc = None if m is None else m.cuda()
    bflags = 0
    o, lse, _, _ = capi.fwd(qc, kc, vc, mask=mc, want_lse=True, **kw)
    dq, dk, dv = capi.bwd(dc, qc, kc, vc, o, lse, mask=mc, flags=bflags, **kw)
    torch.cuda.synchronize()
    if maskk in ("pad", "padinf", "padholes", "keyinf"):
        o2, lse2, _, _ = capi.fwd(qc, kc, vc, mask=mc, want_lse=True, flags=capi.FLAG_NO_MASK_TRIM, **kw)
        g2 = capi.bwd(dc, qc, kc, vc, o, lse, mask=mc, flags=bflags | capi.FLAG_NO_MASK_TRIM, **kw)
        assert torch.equal(o, o2) and torch.equal(lse, lse2), "forward: trimmed != untrimmed"
        if not bflags:
            assert all(torch.equal(x, y) for x, y in zip((dq, dk, dv), g2)), "backward: trimmed != untrimmed"
        else:
            # the one-pass kernel runs full key chunks on a hand-ordered instruction stream and partly
            # filled ones on a plain loop; the two round the same dS element differently now and then
            # (a fused multiply-convert against a multiply followed by a convert): one unit in the last place
            for x, y in zip((dq, dk, dv), g2):
                assert (x.float() - y.float()).abs().max().item() <= 2e-3 * max(1.0, y.float().abs().max().item())
    ref = oracle.attention(f32(q), f32(k), f32(v), mask=mo, dout=f32(do), want=("o", "lse", "dq", "dk", "dv"), **okw)
    otol = (2e-3 if dtype == "fp16" else 2e-2) * max(1.0, float(np.abs(ref["o"]).max()) / 2.0)
    gtol = 1e-2 if dtype == "fp16" else 3e-2
    got_o = f32(o.reshape(bh, sq, d).cpu())
    assert np.abs(got_o - ref["o"]).max() <= otol, "o"
    # the absolute bound for gradients whose true value is zero throughout a head (module docstring): heads of a
    # sequence with one visible key sit beside heads with ordinary gradients, so the two criteria apply head by head
    a_rows = np.abs(f32(do) * got_o).sum(-1)                                   # A_i per (head, query)
    zero_tol = 4 * d ** -0.5 * UNIT[dtype] * np.sqrt((a_rows ** 2).sum(-1)) * \
        float(max(np.abs(f32(q)).max(), np.abs(f32(k)).max()))                 # per head
    for name, t in (("dq", dq), ("dk", dk), ("dv", dv)):
        a = f32(t.reshape(ref[name].shape).cpu())
        assert np.isfinite(a).all(), name
        err = np.abs(a - ref[name]).reshape(bh, -1).max(1)
        top = np.abs(ref[name]).reshape(bh, -1).max(1)
        zero = (top < 1e-6) if name != "dv" else np.zeros(bh, bool)
        assert (err[zero] <= np.maximum(zero_tol[zero], 1e-6)).all(), \
            f"{name}: zero gradient, |got| {err[zero].max():.3e} > {zero_tol[zero].min():.3e}"
        if (~zero).any():
            assert err[~zero].max() / max(top.max(), 1e-3) <= gtol, name
    fin = np.isfinite(ref["lse"])
    gl = lse.reshape(bh, sq).cpu().numpy()
    assert np.array_equal(np.isfinite(gl), fin), "lse: -inf rows differ"
    if fin.any():
        assert np.abs(gl[fin] - ref["lse"][fin]).max() <= 5e-3 + 2.0 ** -8 * np.abs(ref["lse"][fin]).max(), "lse"
    # the same forward with its key range cut into pieces (decode steps take this route by themselves; here it is
    # forced on every third eligible problem): same bars, one more rounding of the partial outputs included
    pr = random.Random(it * 7919 + 13)
    if not causal and not p and maskk != "full" and sk > 128 and pr.random() < 0.34:
        os.environ["FMHA_FWD_SPLIT"] = str(pr.choice([2, 3, 5]))
        try:
            o3, lse3, _, _ = capi.fwd(qc, kc, vc, mask=mc, want_lse=True, **kw)
            torch.cuda.synchronize()
        finally:
            del os.environ["FMHA_FWD_SPLIT"]
        assert np.abs(f32(o3.reshape(bh, sq, d).cpu()) - ref["o"]).max() <= otol, "o in pieces"
        gl3 = lse3.reshape(bh, sq).cpu().numpy()
        assert np.array_equal(np.isfinite(gl3), fin), "lse in pieces: -inf rows differ"
        if fin.any():
            assert np.abs(gl3[fin] - ref["lse"][fin]).max() <= 5e-3 + 2.0 ** -8 * np.abs(ref["lse"][fin]).max(), "lse in pieces"


# problems whose gradients with respect to q and k are zero throughout (every query sees one key)
ZERO_GRADIENT = [
    dict(d=64, dtype="bf16", b=1, h=2, sq=127, sk=1, causal=False, p=0.1, mask="none"),
    dict(d=64, dtype="bf16", b=2, h=1, sq=520, sk=1, causal=True, p=0.0, mask="none"),
    dict(d=128, dtype="fp16", b=1, h=4, sq=257, sk=8, causal=False, p=0.1, mask="padinf", lens=[1], want_strided=True),
    dict(d=64, dtype="fp16", b=2, h=2, sq=300, sk=1, causal=False, p=0.3, mask="full"),
    dict(d=64, dtype="fp16", b=1, h=1, sq=1, sk=200, causal=True, p=0.1, mask="none"),
    dict(d=64, dtype="bf16", b=2, h=2, sq=300, sk=300, causal=False, p=0.1, mask="pad", lens=[1, 1]),
]


@pytest.mark.parametrize("idx", range(len(ZERO_GRADIENT)))
def test_gradients_that_are_exactly_zero(idx):
    rng = random.Random(1000 + idx)
    _run_case(5000 + idx, _case(5000 + idx, rng, dict(ZERO_GRADIENT[idx])), rng)


def test_randomized_sweep_against_the_oracle():
    rng = random.Random(20241125)
    for it in range(400):
        c = _case(it, rng)
        try:
            _run_case(it, c, rng)
        except AssertionError as e:
            raise AssertionError(f"case #{it} {c}: {e}") from e


# ---- the reference's three operators (full [bh,sq,sk] mask tensor; dropout tensor; saved outputs) over sizes that
# reach every kernel they can run on: the one-pass kernel up to 128 keys (and its build for 97 to 128), the streaming
# forward, the one-launch save kernel up to 512 keys, forward + save kernel beyond, and the plain / pipelined kernels
# for key counts that are not multiples of 8.
def _operator_case(it, rng):
    dtype = rng.choice(["fp16", "fp16", "bf16"])
    mode = rng.choice(["infer", "train", "save", "save"])
    bh = rng.choice([1, 2, 5])
    sq = rng.choice([1, 7, 32, 33, 100, 127, 128, 129, 200, 256, 300])
    sk = rng.choice([8, 40, 64, 96, 104, 120, 128, 136, 192, 200, 256, 264, 320, 448, 512, 520, 576, 640, 77, 333])
    maskk = rng.choice(["01", "01", "normal", "infcols"])
    scale = rng.choice([2.0, 1.25, 1.0 / 0.9])
    return dict(dtype=dtype, mode=mode, bh=bh, sq=sq, sk=sk, mask=maskk, drop_scale=scale)


def _run_operator_case(it, c):
    dtype, mode, bh, sq, sk = c["dtype"], c["mode"], c["bh"], c["sq"], c["sk"]
    q, k, v = make_qkv(bh, sq, sk, 64, seed=1000 + it, dtype=dtype)
    g = torch.Generator().manual_seed(2000 + it)
    tol = 2e-3 if dtype == "fp16" else 2e-2
    if mode == "infer":
        m = torch.empty(bh, sq, sk).random_(2, generator=g).to(TDT[dtype])
        o, lse, _, _ = capi.fwd(q.cuda(), k.cuda(), v.cuda(), mask=m.cuda(), mask_kind=capi.MASK_KEEP01, want_lse=True)
        torch.cuda.synchronize()
        ref = oracle.attention(f32(q), f32(k), f32(v), mask=f32(m), mask_kind="keep01", want=("o", "lse"))
        assert np.abs(f32(o.cpu()) - ref["o"]).max() <= tol, "o"
        assert np.abs(lse.cpu().numpy() - ref["lse"]).max() <= (1e-3 if dtype == "fp16" else 5e-3), "lse"
        return
    if c["mask"] == "01":
        pm = torch.empty(bh, sq, sk).random_(2, generator=g) * -1000
    else:
        pm = torch.randn(bh, sq, sk, generator=g) * 2
        if c["mask"] == "infcols":
            pm[:, :, 3::5] = float("-inf")
            pm[:, sq // 2, :] = float("-inf")          # a row that sees no key
            pm[:, 0, : max(1, sk - 3)] = float("-inf")  # a row whose keys are all in the last tile
    pm = pm.to(TDT[dtype])
    dm = torch.empty(bh, sq, sk).random_(2, generator=g).to(TDT[dtype])
    save = mode == "save"
    o, lse, sm, dr = capi.fwd(q.cuda(), k.cuda(), v.cuda(), mask=pm.cuda(), drop_kind=capi.DROP_TENSOR,
                              drop_mask=dm.cuda(), drop_scale=c["drop_scale"], save=save, want_lse=True)
    torch.cuda.synchronize()
    ref = oracle.attention(f32(q), f32(k), f32(v), mask=f32(pm), drop_mask=f32(dm), drop_scale=c["drop_scale"],
                           want=("o", "lse", "softmax", "dropout"))
    got_o = f32(o.cpu())
    assert np.isfinite(got_o).all(), "o not finite"
    assert np.abs(got_o - ref["o"]).max() <= 2 * tol * max(1.0, float(np.abs(ref["o"]).max()) / 2.0), "o"
    dead = np.isneginf(ref["lse"])
    gl = lse.cpu().numpy()
    assert np.array_equal(np.isneginf(gl), dead), "lse: -inf rows differ"
    if (~dead).any():
        assert np.abs(gl[~dead] - ref["lse"][~dead]).max() <= (1e-3 if dtype == "fp16" else 5e-3) * \
            max(1.0, float(np.abs(ref["lse"][~dead]).max()) / 8.0), "lse"
    if save:
        got_sm, got_dr = f32(sm.cpu()), f32(dr.cpu())
        assert np.isfinite(got_sm).all() and np.isfinite(got_dr).all(), "saved outputs not finite"
        assert np.abs(got_sm - ref["softmax"]).max() <= tol / 2, "softmax"
        assert np.abs(got_dr - ref["dropout"]).max() <= tol * max(1.0, c["drop_scale"] / 2.0), "dropout"
        o2, _, _, _ = capi.fwd(q.cuda(), k.cuda(), v.cuda(), mask=pm.cuda(), drop_kind=capi.DROP_TENSOR,
                               drop_mask=dm.cuda(), drop_scale=c["drop_scale"])
        torch.cuda.synchronize()
        if sk % 8 == 0:   # rows on 16-byte boundaries: the saving and the plain call run the same arithmetic
            assert torch.equal(o2, o), "saving changed O"
        else:             # otherwise two kernel families (the plain loop saves, the pipelined loop does not): a unit
            assert (o2.float() - o.float()).abs().max().item() <= tol / 4, "saving changed O"   # in the last place at most


def test_randomized_sweep_of_the_reference_operators():
    rng = random.Random(20241126)
    for it in range(160):
        c = _operator_case(it, rng)
        try:
            _run_operator_case(it, c)
        except AssertionError as e:
            raise AssertionError(f"operator case #{it} {c}: {e}") from e
