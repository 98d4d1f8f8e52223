"""Forward on e4m3 inputs (fmha_fwd_fp8_launch) against the CPU oracle run with the same rounding model:
inputs are the e4m3 values themselves (exact in fp32); the unnormalised probabilities 2^(y - M), y the score in
log2 units and M an INTEGER reference exponent near the row maximum, are rounded to e4m3 before the second
product, and O is that product over the sum of the ROUNDED probabilities.

Tolerances.  e4m3 keeps three mantissa bits: every probability carries a rounding error of up to 2^-4 relative.
Because the reference exponent is an integer, the kernel (whose reference is set by the first tile of a row and
raised lazily) and the oracle (ceil of the row maximum) round the same values up to an exact power of two, so
they round them the same way -- except where a score sits within fp32 rounding of a tie between two e4m3
values, or deep in the subnormal range, which moves single weights by one e4m3 step:
   99.9 % of |O - model| <= 2e-3 * max|v| + rounding of O, all of it <= 2^-4 * max|v|
                                    (kernel and model compute the same thing; a flipped tie in a row of few keys
                                     moves that row by one e4m3 step of one weight)
   rms(O - exact) <= 1.5 * rms(model - exact) + 2^-11 max|O|   (and that thing is as accurate as the format allows)
   max|O - exact| <= 2^-3 * max|v|   (the bound if every probability of a row rounded one way and their sum the other)
   LSE (accumulated from the unrounded probabilities) within 2e-3
where `exact` is the oracle on the same e4m3 inputs without any rounding of the probabilities.  Where nothing
rounds (all probabilities equal, one key per row, one dominant key) the kernel must agree with the oracle to the
rounding of O."""
import numpy as np
import pytest
import torch

import oracle
from nvfuserexamples_amd import capi
from conftest import pad_mask, f32

pytestmark = pytest.mark.gpu

CASES = [
    # bh, sq, sk, d, out dtype, mask, causal
    (4, 128, 128, 64, torch.float16, None, False),
    (4, 512, 512, 64, torch.float16, "pad", False),     # headline shape, few heads
    (3, 100, 77, 64, torch.float16, None, False),        # ragged tiles
    (2, 320, 320, 64, torch.float16, None, True),        # causal
    (2, 200, 333, 128, torch.bfloat16, "pad", False),
    (2, 257, 257, 128, torch.float16, "pad", True),
    (2, 1, 1000, 64, torch.float16, None, False),        # one query row (kept on this kernel: FMHA_FWD_DECODE=0)
]


@pytest.fixture
def matrix_pipe_only(monkeypatch):
    """Keeps launches of one to four query rows off the decode kernel, whose probabilities stay fp32."""
    monkeypatch.setenv("FMHA_FWD_DECODE", "0")
    yield
    monkeypatch.delenv("FMHA_FWD_DECODE")
    capi.lib().fmha_reload_overrides()


def _quantise(x, amax=448.0):
    """Per-tensor scaling into the e4m3 range; returns (e4m3 tensor, dequantisation factor)."""
    s = float(x.abs().max()) / amax
    return (x / s).to(torch.float8_e4m3fn), s


@pytest.mark.parametrize("bh,sq,sk,d,odt,mask,causal", CASES)
def test_fp8_forward_matches_the_oracle_with_the_same_rounding(bh, sq, sk, d, odt, mask, causal, matrix_pipe_only):
    g = torch.Generator().manual_seed(bh + sk)
    std = 1.0 if d == 64 else 0.5
    q, k, v = (torch.randn(bh, s, d, generator=g) * std for s in (sq, sk, sk))
    q8, dq = _quantise(q)
    k8, dk = _quantise(k)
    v8, dv = _quantise(v)
    m = None
    if mask == "pad":
        m = pad_mask(bh // 2 if bh % 2 == 0 else bh, sk, sk // 2, sk).to(odt)
    o, lse = capi.fwd_fp8(q8.cuda(), k8.cuda(), v8.cuda(), dq, dk, dv, mask=None if m is None else m.cuda(),
                          causal=causal, out_dtype=odt, want_lse=True)
    torch.cuda.synchronize()
    qf, kf, vf = (f32(t.float()) for t in (q8, k8, v8))   # the e4m3 values, exactly
    kw = dict(mask=None if m is None else f32(m), causal=causal, scale=d ** -0.5 * dq * dk, want=("o", "lse"))
    ref = oracle.attention(qf, kf, vf * np.float32(dv), round_p="e4m3", **kw)
    exact = oracle.attention(qf, kf, vf * np.float32(dv), **kw)
    got = f32(o.cpu())
    top = np.abs(exact["o"]).max()
    out_round = 2.0 ** -11 if odt == torch.float16 else 2.0 ** -8
    rms = lambda x: float(np.sqrt(np.mean(np.square(x, dtype=np.float64))))
    dev = np.abs(got - ref["o"])
    vmax = float(np.abs(vf).max()) * dv
    assert np.quantile(dev, 0.999) <= 2e-3 * vmax + out_round * top
    assert dev.max() <= 2.0 ** -4 * vmax + out_round * top
    assert rms(got - exact["o"]) <= 1.5 * rms(ref["o"] - exact["o"]) + out_round * top
    assert np.abs(got - exact["o"]).max() <= 2.0 ** -3 * float(np.abs(vf).max()) * dv + out_round * top
    assert np.abs(lse.cpu().numpy() - ref["lse"]).max() <= 2e-3
    # and the 8-bit path is a different computation from a cast of the 16-bit one: the model's rounding shows
    assert np.abs(ref["o"] - exact["o"]).max() > 1e-4 * top


@pytest.mark.parametrize("bh,sq,sk,d,causal", [(4, 100, 700, 64, False), (2, 257, 512, 128, True)])
def test_fp8_peaked_rows_and_moving_references(bh, sq, sk, d, causal):
    """Scores sixteen times larger: a row's weight sits on one or two keys, its maximum differs by tens of
    binades from tile to tile, so the reference exponent is raised (and everything rescaled by the exact power
    of two) again and again.  A flipped tie now moves a whole row by one e4m3 step of a dominant weight, and the
    kernel's reference may sit up to eight binades below the model's ceil(max), which keeps probabilities the
    model flushes on e4m3's subnormal grid (below 2^-6 of the row maximum: 2^-10 of it each, hundreds of keys).
    So the comparison with the model is made per row -- all but a few rows agree to 1e-2 of max|v|, every row
    to one step -- and against the unrounded result the kernel must be no worse than the model."""
    g = torch.Generator().manual_seed(sk)
    std = 4.0 if d == 64 else 2.0
    q, k, v = (torch.randn(bh, s, d, generator=g) * std for s in (sq, sk, sk))
    q8, dq = _quantise(q)
    k8, dk = _quantise(k)
    v8, dv = _quantise(v)
    m = pad_mask(bh, sk, sk // 2, sk).half()
    o, lse = capi.fwd_fp8(q8.cuda(), k8.cuda(), v8.cuda(), dq, dk, dv, mask=m.cuda(), causal=causal, want_lse=True)
    torch.cuda.synchronize()
    qf, kf, vf = (f32(t.float()) for t in (q8, k8, v8))
    kw = dict(mask=f32(m), causal=causal, scale=d ** -0.5 * dq * dk, want=("o", "lse"))
    ref = oracle.attention(qf, kf, vf * np.float32(dv), round_p="e4m3", **kw)
    exact = oracle.attention(qf, kf, vf * np.float32(dv), **kw)
    got = f32(o.cpu())
    assert np.isfinite(got).all()
    vmax = float(np.abs(vf).max()) * dv
    rowdev = np.abs(got - ref["o"]).max(-1) / vmax
    assert (rowdev > 1e-2).mean() <= 0.03
    assert rowdev.max() <= 2.0 ** -4 + 1e-3
    rms = lambda x: float(np.sqrt(np.mean(np.square(x, dtype=np.float64))))
    assert rms(got - exact["o"]) <= 1.1 * rms(ref["o"] - exact["o"]) + 2.0 ** -11 * float(np.abs(exact["o"]).max())
    assert np.abs(lse.cpu().numpy() - ref["lse"]).max() <= 3e-3


@pytest.mark.parametrize("d,odt", [(64, torch.float16), (128, torch.bfloat16)])
def test_fp8_forward_is_exact_where_nothing_rounds(d, odt):
    """q = 0: every probability is 1 (an e4m3 value), O is the mean of the e4m3 values of v.  One-hot q and k
    with a score gap of 100: one probability is 1, the others underflow to 0, O_i = v[i mod d] -- which also
    pins the key <-> register permutation of the first product and the transposed V tile, element by element."""
    g = torch.Generator().manual_seed(d)
    bh, sq, sk = 3, 200, 333
    v = torch.randn(bh, sk, d, generator=g)
    v8 = v.to(torch.float8_e4m3fn)
    q8 = torch.zeros(bh, sq, d).to(torch.float8_e4m3fn)
    k8 = torch.randn(bh, sk, d, generator=g).to(torch.float8_e4m3fn)
    o, lse = capi.fwd_fp8(q8.cuda(), k8.cuda(), v8.cuda(), descale_v=0.5, out_dtype=odt, want_lse=True)
    want = 0.5 * v8.float().mean(1, keepdim=True).expand(bh, sq, d)
    tol = (2.0 ** -10 if odt == torch.float16 else 2.0 ** -7) * float(want.abs().max()) + 1e-6
    assert (o.float().cpu() - want).abs().max().item() <= tol
    assert (lse.cpu() - np.log(sk)).abs().max().item() <= 1e-5
    sq = sk = d                                   # one key per query matches
    eye = torch.eye(d).expand(bh, d, d) * 16.0    # 16 * 16 * (100 / 256) = 100
    e8 = eye.contiguous().to(torch.float8_e4m3fn)
    vv = torch.randn(bh, sk, d, generator=g).to(torch.float8_e4m3fn)
    o, _ = capi.fwd_fp8(e8.cuda(), e8.cuda(), vv.cuda(), scale=100.0 / 256.0, out_dtype=odt)
    assert torch.equal(o.float().cpu(), vv.float().to(odt).float())


def test_fp8_forward_refuses_what_it_does_not_serve():
    x = torch.zeros(2, 64, 96, device="cuda").to(torch.float8_e4m3fn)
    with pytest.raises(capi.FmhaError):
        capi.fwd_fp8(x, x, x)                                   # head dim 96
    y = torch.zeros(2, 64, 64, device="cuda").to(torch.float8_e4m3fn)
    with pytest.raises(capi.FmhaError):
        capi.fwd_fp8(y, y, y, descale_q=0.0)                    # a factor must be positive
    with pytest.raises(capi.FmhaError):
        capi.fwd_fp8(y, y, y, mask=torch.zeros(2, 64, 64, dtype=torch.float16, device="cuda"))  # per-key masks only


def test_fp8_operator_equals_the_c_abi_call():
    from nvfuserexamples_amd import load_ops
    ops = load_ops()
    g = torch.Generator().manual_seed(1)
    q8, k8, v8 = (torch.randn(4, 160, 64, generator=g).to(torch.float8_e4m3fn).cuda() for _ in range(3))
    m = pad_mask(2, 160, 80, 160).half().cuda()
    o, lse = ops.fmha_fwd_fp8(q8, k8, v8, 0.5, 2.0, 1.5, m, 0.0, False)
    o2, lse2 = capi.fwd_fp8(q8, k8, v8, 0.5, 2.0, 1.5, mask=m, want_lse=True)
    assert torch.equal(o, o2) and torch.equal(lse, lse2)


DECODE_CASES = [
    # bh, sq, sk, d, out dtype, mask, kv_len, forced pieces (None: the library's choice, 0: never)
    (4, 1, 1000, 64, torch.float16, None, False, 0),
    (2, 1, 4096, 128, torch.float16, None, False, None),     # cut by the library itself
    (4, 2, 3000, 128, torch.bfloat16, "pad", True, 3),
    (3, 4, 700, 64, torch.float16, None, True, 2),
    (2, 3, 333, 128, torch.float16, "pad", False, 0),
]


@pytest.mark.parametrize("bh,sq,sk,d,odt,mask,kvl,force", DECODE_CASES)
def test_fp8_decode_steps_keep_fp32_probabilities(bh, sq, sk, d, odt, mask, kvl, force, monkeypatch):
    """One to four query rows without a causal mask run on the streaming decode kernel: e4m3 rows are unpacked to
    fp32 and nothing is rounded until O, so the result is the oracle's on the same e4m3 inputs WITHOUT any rounding
    of the probabilities, to the rounding of O (plus 1e-4 of max|v| for the fp32 sums); valid key counts and the key
    range in pieces as in the 16-bit forward."""
    g = torch.Generator().manual_seed(bh * 100 + sk)
    std = 1.0 if d == 64 else 0.5
    q, k, v = (torch.randn(bh, s, d, generator=g) * std for s in (sq, sk, sk))
    q8, dq = _quantise(q)
    k8, dk = _quantise(k)
    v8, dv = _quantise(v)
    m = pad_mask(bh // 2 if bh % 2 == 0 else bh, sk, sk // 2, sk).to(odt) if mask == "pad" else None
    lens = torch.randint(1, sk + 1, (bh,), generator=g, dtype=torch.int32) if kvl else None
    if force is not None:
        monkeypatch.setenv("FMHA_FWD_SPLIT", str(force))
    try:
        o, lse = capi.fwd_fp8(q8.cuda(), k8.cuda(), v8.cuda(), dq, dk, dv, mask=None if m is None else m.cuda(),
                              out_dtype=odt, want_lse=True, kv_len=None if lens is None else lens.cuda())
        o0, lse0 = capi.fwd_fp8(q8.cuda(), k8.cuda(), v8.cuda(), dq, dk, dv, mask=None if m is None else m.cuda(),
                                out_dtype=odt, want_lse=True, kv_len=None if lens is None else lens.cuda(),
                                workspace=False)
        torch.cuda.synchronize()
    finally:
        monkeypatch.delenv("FMHA_FWD_SPLIT", raising=False)
        capi.lib().fmha_reload_overrides()
    full = np.zeros((bh, sq, sk), np.float32)
    if m is not None:
        full += np.repeat(f32(m).reshape(-1, 1, sk), bh // m.shape[0], 0)
    if lens is not None:
        for i, n in enumerate(lens.tolist()):
            full[i, :, n:] = -np.inf
    qf, kf, vf = (f32(t.float()) for t in (q8, k8, v8))
    exact = oracle.attention(qf, kf, vf * np.float32(dv), mask=full, scale=d ** -0.5 * dq * dk, want=("o", "lse"))
    top = np.abs(exact["o"]).max()
    vmax = float(np.abs(vf).max()) * dv
    out_round = 2.0 ** -11 if odt == torch.float16 else 2.0 ** -8
    for got, gl in ((o, lse), (o0, lse0)):
        assert np.abs(f32(got.cpu()) - exact["o"]).max() <= 1e-4 * vmax + out_round * top
        assert np.abs(gl.cpu().numpy() - exact["lse"]).max() <= 1e-3


def test_fp8_key_counts_need_the_decode_kernel():
    """Launches the decode kernel does not serve (more than four rows, causal) refuse valid key counts."""
    q8, k8, v8 = (torch.randn(2, s, 64).to(torch.float8_e4m3fn).cuda() for s in (8, 256, 256))
    lens = torch.tensor([100, 200], dtype=torch.int32).cuda()
    with pytest.raises(capi.FmhaError, match="-6"):
        capi.fwd_fp8(q8, k8, v8, kv_len=lens)
