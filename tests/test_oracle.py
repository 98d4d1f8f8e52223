"""Pins the CPU oracle (``oracle/``) without a GPU.

The reference holds no golden vectors (its tests compare fused vs eager on fresh
random inputs: test.py:20-29, test_train_mha.py:23-41), so every function of the
oracle is pinned by an independent statement of the same mathematics:
library matmul/softmax compositions, closed forms and invariants, the Random123
known-answer vectors for Philox, and finite differences / autograd for the backward.
"""
import numpy as np
import pytest
import torch

import oracle
from oracle import eager
from conftest import make_qkv, pad_mask, f32, rel_to_max


# ------------------------------------------------------------------ Philox

# Random123 kat_vectors for philox4x32-10: (counter, key) -> output
PHILOX_KAT = [
    ([0, 0, 0, 0], [0, 0], [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]),
    ([0xffffffff] * 4, [0xffffffff] * 2, [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]),
    ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0],
     [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]),
]


@pytest.mark.parametrize("ctr,key,want", PHILOX_KAT)
def test_philox_known_answers(ctr, key, want):
    assert [int(x) for x in oracle.philox4x32_10(ctr, key)] == want


def _philox_py(ctr, key):
    """Independent pure-Python statement of the published round function."""
    c, k = list(ctr), list(key)
    for _ in range(10):
        p0, p1 = 0xD2511F53 * c[0], 0xCD9E8D57 * c[2]
        c = [((p1 >> 32) ^ c[1] ^ k[0]) & 0xffffffff, p1 & 0xffffffff,
             ((p0 >> 32) ^ c[3] ^ k[1]) & 0xffffffff, p0 & 0xffffffff]
        k = [(k[0] + 0x9E3779B9) & 0xffffffff, (k[1] + 0xBB67AE85) & 0xffffffff]
    return c


def test_keep_rule_matches_definition():
    """keep(bh,q,k) == byte (q%4, k%4) of the Philox block of the 4x4 tile >= threshold."""
    seed, offset, p = 0x123456789abcdef, 0x1122334455, 0.3
    bh, sq, sk = 3, 10, 13
    km = oracle.keep_mask(seed, offset, p, bh, sq, sk)
    thr = oracle.drop_threshold(p)
    assert thr == 77  # round(0.3*256)
    qb4, kb4 = (sq + 3) // 4, (sk + 3) // 4
    for b in range(bh):
        for q in range(sq):
            for k in range(sk):
                blk = (b * qb4 + q // 4) * kb4 + k // 4
                out = _philox_py([offset & 0xffffffff, offset >> 32, blk & 0xffffffff, blk >> 32],
                                 [seed & 0xffffffff, seed >> 32])
                byte = (out[q % 4] >> (8 * (k % 4))) & 0xff
                assert km[b, q, k] == (byte >= thr)


def test_keep_rule_statistics_and_streams():
    km = oracle.keep_mask(1, 0, 0.1, 4, 128, 128)
    assert abs(km.mean() - (1 - 26 / 256)) < 5e-3          # threshold 26/256
    assert oracle.keep_mask(1, 0, 0.0, 1, 8, 8).all()        # p = 0 keeps everything
    assert (oracle.keep_mask(1, 0, 0.1, 4, 128, 128) == km).all()  # deterministic
    other = oracle.keep_mask(1, 1, 0.1, 4, 128, 128)         # next offset: fresh stream
    assert 0.75 < (other == km).mean() < 0.9
    assert [oracle.drop_threshold(p) for p in (0.0, 0.1, 0.5, 0.999)] == [0, 26, 128, 255]


# ------------------------------------------------------------------ rounding

@pytest.mark.parametrize("kind,tdt", [("fp16", torch.float16), ("bf16", torch.bfloat16)])
def test_rounding_matches_torch_casts(kind, tdt):
    g = torch.Generator().manual_seed(3)
    x = torch.cat([torch.randn(4000, generator=g) * s for s in (1e-7, 1e-5, 1e-3, 1.0, 300.0, 7e4)])
    want = x.to(tdt).float().numpy()
    got = np.array([oracle.lib().fmha_oracle_round(float(v), oracle.ROUND[kind]) for v in x.numpy()],
                   dtype=np.float32)
    assert np.array_equal(got, want)


# ------------------------------------------------------------------ forward

def test_inference_matches_eager_composition():
    """Reference test.py:12-18 semantics at its CPU-sized case (B8 H12 S128 D64)."""
    q, k, v = make_qkv(96, 128, 128, 64, seed=0)
    g = torch.Generator().manual_seed(5)
    amask = torch.empty(96, 128, 128).random_(2, generator=g)
    want = eager.infer_mha(q, k, v, amask)
    got = oracle.attention(f32(q), f32(k), f32(v), mask=amask.numpy(), mask_kind="keep01")["o"]
    assert np.abs(got - want.numpy()).max() < 2e-5
    # and with the [B,1,1,S] padding-mask layout
    pm = pad_mask(8, 128, 64, 128)
    want = eager.general_mha(q, k, v, add_mask=pm.expand(8, 12, 1, 128).reshape(96, 1, 128), dtype=torch.float64)
    got = oracle.attention(f32(q), f32(k), f32(v), mask=pm.numpy())["o"]
    assert np.abs(got - want.numpy()).max() < 1e-5


def test_train_matches_eager_composition_and_saved_outputs():
    """Reference test_train_mha.py:14-21: (softmax, dropped, ctx); kept entries scaled by 1/0.5."""
    bh, s, d = 6, 64, 64
    q, k, v = make_qkv(bh, s, s, d, seed=2)
    g = torch.Generator().manual_seed(7)
    pm = torch.empty(bh, s, s).random_(2, generator=g) * -1000.0
    dm = torch.empty(bh, s, s).random_(2, generator=g)
    sm, dr, ctx = eager.train_mha(q, k, v, pm, dm, keep_prob=0.5, dtype=torch.float64)
    got = oracle.attention(f32(q), f32(k), f32(v), mask=pm.numpy(), drop_mask=dm.numpy(), drop_scale=2.0,
                           want=("o", "softmax", "dropout", "lse"))
    assert np.abs(got["o"] - ctx.numpy()).max() < 1e-5
    assert np.abs(got["softmax"] - sm.numpy()).max() < 1e-6
    assert np.abs(got["dropout"] - dr.numpy()).max() < 1e-6
    # zero pattern of the dropped output is the zero pattern of the mask wherever P > 0
    assert np.array_equal(got["dropout"][got["softmax"] > 0] == 0, (dm.numpy() == 0)[got["softmax"] > 0])
    s_ = (q.double() @ k.double().transpose(1, 2)) / 8 + pm.double()
    assert np.abs(got["lse"] - torch.logsumexp(s_, -1).numpy()).max() < 1e-5


def test_forward_closed_forms():
    bh, s, d = 4, 48, 64
    q, k, v = make_qkv(bh, s, s, d, seed=9)
    base = oracle.attention(f32(q), f32(k), f32(v), want=("o", "softmax"))
    ones = np.ones((bh, s, s), np.float32)
    # keep-everything 0/1 mask and all-zero additive mask are no-ops
    assert np.array_equal(oracle.attention(f32(q), f32(k), f32(v), mask=ones, mask_kind="keep01")["o"], base["o"])
    assert np.array_equal(oracle.attention(f32(q), f32(k), f32(v), mask=0 * ones)["o"], base["o"])
    # a whole row masked with a finite constant is a shift: softmax unchanged (fmha_manual.cpp:70)
    row = 0 * ones
    row[:, 5, :] = -10000.0
    np.testing.assert_allclose(oracle.attention(f32(q), f32(k), f32(v), mask=row)["o"], base["o"], atol=1e-6)
    # masked columns get (numerically) zero probability
    col = 0 * ones
    col[:, :, 7] = -10000.0
    assert oracle.attention(f32(q), f32(k), f32(v), mask=col, want=("softmax",))["softmax"][:, :, 7].max() == 0.0
    # rows sum to one, probabilities non-negative
    np.testing.assert_allclose(base["softmax"].sum(-1), 1.0, atol=1e-6)
    assert base["softmax"].min() >= 0
    # legacy dropout: mask of ones doubles the output, mask of zeros kills it
    np.testing.assert_allclose(
        oracle.attention(f32(q), f32(k), f32(v), drop_mask=ones, drop_scale=2.0)["o"], 2 * base["o"], rtol=1e-6)
    assert not oracle.attention(f32(q), f32(k), f32(v), drop_mask=0 * ones, drop_scale=2.0)["o"].any()
    # one key: output is that key's value row
    o1 = oracle.attention(f32(q), f32(k[:, :1]), f32(v[:, :1]))["o"]
    np.testing.assert_allclose(o1, np.broadcast_to(f32(v[:, :1]), o1.shape), atol=1e-7)
    # q = 0: uniform average of v
    ou = oracle.attention(0 * f32(q), f32(k), f32(v))["o"]
    np.testing.assert_allclose(ou, np.broadcast_to(f32(v).mean(1, keepdims=True), ou.shape), atol=1e-6)


def test_causal_and_philox_match_eager():
    bh, sq, sk, d = 3, 40, 40, 64
    q, k, v = make_qkv(bh, sq, sk, d, seed=4)
    want = eager.general_mha(q, k, v, causal=True, dtype=torch.float64).numpy()
    got = oracle.attention(f32(q), f32(k), f32(v), causal=True)["o"]
    assert np.abs(got - want).max() < 1e-5
    keep = torch.from_numpy(oracle.keep_mask(11, 3, 0.25, bh, sq, sk).astype(np.float32))
    want = eager.general_mha(q, k, v, causal=True, keep=keep, drop_scale=1 / 0.75, dtype=torch.float64).numpy()
    got = oracle.attention(f32(q), f32(k), f32(v), causal=True, philox=True, p_drop=0.25, drop_scale=1 / 0.75,
                           seed=11, offset=3)["o"]
    assert np.abs(got - want).max() < 1e-5


def test_p_rounding_point_is_small_and_modelled():
    """Rounding P to half before P.V (fmha_manual.cpp:87) moves O by well under the parity budget."""
    q, k, v = make_qkv(4, 128, 128, 64, seed=6)
    a = oracle.attention(f32(q), f32(k), f32(v))["o"]
    b = oracle.attention(f32(q), f32(k), f32(v), round_p="fp16")["o"]
    assert 0 < np.abs(a - b).max() < 5e-4


# ------------------------------------------------------------------ backward

def _autograd_grads(q, k, v, do, **kw):
    q, k, v = (t.double().requires_grad_(True) for t in (q, k, v))
    o = eager.general_mha(q, k, v, dtype=torch.float64, **kw)
    o.backward(do.double())
    return q.grad.numpy(), k.grad.numpy(), v.grad.numpy()


@pytest.mark.parametrize("case", ["plain", "mask", "causal", "philox", "ragged"])
def test_backward_matches_autograd(case):
    bh, sq, sk, d = 3, 24, 24, 64
    if case == "ragged":
        sq, sk = 19, 29
    q, k, v, do = make_qkv(bh, sq, sk, d, seed=12, with_dout=True)
    kw, okw = {}, {}
    if case == "mask":
        g = torch.Generator().manual_seed(1)
        m = torch.randn(bh, sq, sk, generator=g)
        kw["add_mask"], okw["mask"] = m, m.numpy()
    if case == "causal":
        kw["causal"] = okw["causal"] = True
    if case == "philox":
        keep = torch.from_numpy(oracle.keep_mask(5, 9, 0.2, bh, sq, sk).astype(np.float32))
        kw.update(keep=keep, drop_scale=1.25)
        okw.update(philox=True, p_drop=0.2, drop_scale=1.25, seed=5, offset=9)
    want = _autograd_grads(q, k, v, do, **kw)
    got = oracle.attention(f32(q), f32(k), f32(v), dout=f32(do), want=("dq", "dk", "dv"), **okw)
    for w, name in zip(want, ("dq", "dk", "dv")):
        assert rel_to_max(got[name], w) < 1e-5, name


def test_backward_finite_differences():
    """Central differences in fp64 on a tiny case: a dropped term or wrong sign fails this."""
    bh, sq, sk, d = 2, 8, 8, 4
    rng = np.random.default_rng(0)
    q, k, v, do = (rng.standard_normal((bh, s, d)).astype(np.float32) for s in (sq, sk, sk, sq))
    mask = rng.standard_normal((bh, sq, sk)).astype(np.float32)
    kw = dict(mask=mask, scale=0.5, philox=True, p_drop=0.3, drop_scale=1 / 0.7, seed=3, offset=1)
    got = oracle.attention(q, k, v, dout=do, want=("dq", "dk", "dv"), **kw)

    def loss(q_, k_, v_):
        return float((oracle.attention(q_, k_, v_, **kw)["o"].astype(np.float64) * do).sum())

    eps = 1e-2
    for name, idx in (("dq", 0), ("dk", 1), ("dv", 2)):
        arrs = [q, k, v]
        num = np.zeros_like(arrs[idx], dtype=np.float64)
        it = np.nditer(arrs[idx], flags=["multi_index"])
        for _ in it:
            i = it.multi_index
            save = arrs[idx][i]
            arrs[idx][i] = save + eps
            lp = loss(*arrs)
            arrs[idx][i] = save - eps
            lm = loss(*arrs)
            arrs[idx][i] = save
            num[i] = (lp - lm) / (2 * eps)
        assert rel_to_max(got[name], num) < 2e-3, name


def test_backward_invariants():
    bh, s, d = 2, 16, 64
    q, k, v, do = make_qkv(bh, s, s, d, seed=21, with_dout=True)
    # p = 0 Philox path is the no-dropout path
    a = oracle.attention(f32(q), f32(k), f32(v), dout=f32(do), want=("dq", "dk", "dv"))
    b = oracle.attention(f32(q), f32(k), f32(v), dout=f32(do), want=("dq", "dk", "dv"), philox=True, p_drop=0.0,
                         drop_scale=1.0, seed=4)
    for n in a:
        assert np.array_equal(a[n], b[n])
    # dV = P^T dO when nothing is dropped
    p = oracle.attention(f32(q), f32(k), f32(v), want=("softmax",))["softmax"].astype(np.float64)
    np.testing.assert_allclose(a["dv"], np.einsum("bqk,bqd->bkd", p, f32(do).astype(np.float64)), atol=1e-5)


@pytest.mark.parametrize("p", [0.001, 0.1, 0.3, 0.5, 0.9])
def test_dropout_factor_keeps_the_mean(p):
    """Kept values are scaled by the reciprocal of the keep probability that the 8-bit threshold
    realises, not of the nominal 1 - p: (256 - thr) / 256 * scale == 1 exactly, and the sample mean of
    keep * scale over 2.6 million decisions is 1 within 4 sigma.  A threshold of 0 (p < 1/512) drops
    nothing and scales nothing."""
    thr, scale = oracle.drop_threshold(p), oracle.drop_scale(p)
    assert thr == int(np.floor(p * 256 + 0.5))
    assert (256 - thr) / 256 * scale == pytest.approx(1.0, abs=1e-7)
    if thr == 0:
        assert scale == 1.0 and oracle.keep_mask(3, 1, p, 2, 16, 16).all()
        return
    km = oracle.keep_mask(7, 11, p, 10, 512, 512)
    pk = (256 - thr) / 256
    sigma = np.sqrt(pk * (1 - pk) / km.size) * scale
    assert abs(km.mean() * scale - 1.0) <= 4 * sigma
    # the nominal factor 1 / (1 - p) is biased wherever 256 p is not an integer: by -0.17 % at p = 0.1 (8 sigma here)
    if p == 0.1:
        assert abs(km.mean() / (1 - p) - 1.0) > 4 * sigma


def test_e4m3_rounding_matches_the_library_cast():
    """The oracle's e4m3 rounding (the model of the 8-bit forward) against torch's float8_e4m3fn cast:
    a dense sweep of the finite range, the subnormal region and the ties, bit for bit."""
    x = torch.cat([torch.linspace(-448, 448, 60001), torch.randn(20000) * 0.01, torch.randn(20000),
                   torch.tensor([0.0, 2.0 ** -9, 2.0 ** -10, 1.5 * 2.0 ** -9, 448.0, 447.0, 0.0155, 0.0157,
                                 0.9375, 0.96875, 1.0625, 1.1875])])
    want = x.to(torch.float8_e4m3fn).float().numpy()
    got = oracle.round_to(x.numpy(), "e4m3")
    assert np.array_equal(got, want)


def test_e4m3_probability_model_reduces_to_the_exact_forward_when_nothing_rounds():
    """With one key per row the weight is P~ / P~ = 1 whatever the rounding did: the 8-bit model equals the
    unrounded forward.  The same holds for a row with one dominant key (the others underflow e4m3).  With more
    keys it differs, by at most 2^-4 relative per probability and as much again for their sum."""
    q, k, v = make_qkv(2, 9, 1, 64, seed=5)
    a = oracle.attention(f32(q), f32(k), f32(v), round_p="e4m3")["o"]
    b = oracle.attention(f32(q), f32(k), f32(v))["o"]
    assert np.array_equal(a, b)
    eye = np.eye(16, dtype=np.float32)[None] * 10.0           # q_i . k_j = 100 [i == j]: gaps of 100 / 4 nats
    vv = f32(make_qkv(1, 16, 16, 16, seed=7)[2])
    a = oracle.attention(eye, eye, vv, round_p="e4m3", scale=0.25)["o"]
    assert np.array_equal(a, vv)
    q, k, v = make_qkv(2, 16, 40, 64, seed=6)
    a = oracle.attention(f32(q), f32(k), f32(v), round_p="e4m3")["o"]
    b = oracle.attention(f32(q), f32(k), f32(v))["o"]
    assert 0 < np.abs(a - b).max() <= 2.0 ** -3 * np.abs(f32(v)).max()


def test_e4m3_probability_model_against_a_restatement_on_the_library_cast():
    """The model, restated with torch's own float8_e4m3fn cast as the rounding: P~ = e4m3(2^(y - ceil(max y))) with
    y the scores in log2 units, O = P~ v / sum P~.  Any integer reference gives the same weights except in the
    subnormal range (below 2^-6, where e4m3 rounds on a fixed grid of 2^-9): with the reference 3 lower, values are
    8 times larger (still far below 448) and only probabilities below 2^-6 of the row maximum may round differently,
    each by at most 2^-10 of it."""
    q, k, v = (f32(t) for t in make_qkv(3, 20, 50, 32, seed=8))
    got = oracle.attention(q, k, v, round_p="e4m3")["o"]
    y = torch.from_numpy(q).double() @ torch.from_numpy(k).double().transpose(1, 2) * float(np.float32(32 ** -0.5)) * np.log2(np.e)
    for shift, tol in ((0.0, 1e-6), (3.0, 50 * 2.0 ** -10)):
        m = torch.ceil(y.amax(-1, keepdim=True)) - shift
        pt = torch.exp2(y - m).float().to(torch.float8_e4m3fn).double()
        want = (pt @ torch.from_numpy(v).double()) / pt.sum(-1, keepdim=True)
        assert np.abs(got - want.numpy()).max() <= tol * np.abs(v).max()
