"""Decode steps and other launches with few heads, few query rows and a long key range: the forward
cuts the key range into pieces that run as heads of their own and merges them (`workspace` of the
forward's parameter block; no counterpart in the reference, whose shapes are fixed at 128 x 128
per head, reference fmha/fmha_manual.cpp:24-29).

Checked against the CPU oracle on the whole key range (same tolerances as the other forward tests)
and against this build's own plain launch: the pieces' outputs are rounded to the element type once
more before the merge, so the two agree to a little over one rounding of that type, not bit for bit.
FMHA_FWD_SPLIT=n forces about n pieces, so that small shapes exercise ragged last pieces, pieces a
valid-key count leaves empty, masks and run-time layouts.
"""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
from nvfuserexamples_amd import capi
from conftest import make_qkv, f32

pytestmark = pytest.mark.gpu

O_TOL = {"fp16": 2e-3, "bf16": 2e-2}
SELF_TOL = {"fp16": 1.5e-3, "bf16": 1.2e-2}   # one more rounding of values up to ~1: 2^-11 resp. 2^-8, both ways
STD = {64: 1.0, 96: 0.7, 128: 0.5, 200: 0.35, 256: 0.35}


@pytest.fixture
def pieces(monkeypatch):
    """force(n): about n pieces (None: the library's own choice); force(n, decode_kernel=False) also keeps
    launches of one to four query rows off the decode kernel, on the matrix-pipe kernels."""
    def force(n, decode_kernel=True):
        if n is None:
            monkeypatch.delenv("FMHA_FWD_SPLIT", raising=False)
        else:
            monkeypatch.setenv("FMHA_FWD_SPLIT", str(n))
        if decode_kernel:
            monkeypatch.delenv("FMHA_FWD_DECODE", raising=False)
        else:
            monkeypatch.setenv("FMHA_FWD_DECODE", "0")
    yield force
    monkeypatch.delenv("FMHA_FWD_SPLIT", raising=False)
    monkeypatch.delenv("FMHA_FWD_DECODE", raising=False)
    capi.lib().fmha_reload_overrides()


def _params(bh, sq, sk, d, **kw):
    P = capi.FwdParams()
    P.bh, P.sq, P.sk, P.d = bh, sq, sk, d
    P.scale = d ** -0.5
    for k, v in kw.items():
        setattr(P, k, v)
    return P


CASES = [
    # bh, sq, sk, d, dtype, forced pieces (None = the library's own choice), mask, kv_len
    (4, 1, 4096, 64, "fp16", None, None, False),       # a decode step: chosen by the library itself
    (2, 1, 8192, 128, "bf16", None, None, False),
    (3, 1, 1000, 64, "fp16", 3, None, False),          # ragged last piece (384 + 384 + 232)
    (3, 5, 700, 128, "fp16", 4, None, True),           # counts that leave pieces partly and wholly empty
    (4, 1, 640, 64, "bf16", 5, "pad", False),          # per-key padding mask [B,1,1,sk]
    (4, 3, 900, 64, "fp16", 3, "perhead", True),       # per-head [bh,1,sk] mask with holes, and counts
    (2, 130, 520, 64, "fp16", 2, None, False),         # two query tiles per head
    (2, 1, 1500, 96, "fp16", 4, None, False),          # a head dim between the built ones
    (2, 2, 1100, 256, "bf16", 3, "pad", True),         # head dim 256: the plain forward loop
    (2, 1, 2048, 64, "fp16", 64, None, False),         # as many pieces as there are 128-key runs
    (5, 2, 777, 128, "bf16", 2, "perhead", True),      # two query rows
    (4, 4, 1234, 64, "fp16", 3, "pad", True),          # four
    (3, 3, 333, 128, "fp16", 2, None, False),          # three (run as four)
    (3, 8, 900, 128, "bf16", 3, "perhead", True),      # eight rows: the matrix-pipe kernels on the pieces
    (2, 6, 1100, 64, "fp16", 2, "pad", False),
]


def _inputs(bh, sq, sk, d, dtype, mask, kvl, seed):
    q, k, v = make_qkv(bh, sq, sk, d, seed=seed, std=STD[d], dtype=dtype)
    g = torch.Generator().manual_seed(seed + 7)
    m = lens = None
    if mask == "pad":
        b = 2
        m = torch.zeros(b, 1, 1, sk)
        for i, n in enumerate(torch.randint(sk // 3, sk + 1, (b,), generator=g).tolist()):
            m[i, ..., n:] = -10000.0
    elif mask == "perhead":
        m = torch.zeros(bh, 1, sk)
        m[torch.rand(bh, 1, sk, generator=g) < 0.3] = float("-inf")
        m[..., 0] = 0.0
    if kvl:
        lens = torch.randint(1, sk + 1, (bh,), generator=g, dtype=torch.int32)
        lens[0] = min(sk, 130)  # leaves every piece but the first (two) empty
    return q, k, v, m, lens


def _oracle_mask(m, lens, bh, sq, sk):
    full = torch.zeros(bh, sq, sk)
    if m is not None:
        mm = m.reshape(m.shape[0], 1, sk).float()
        full = full + mm.repeat_interleave(bh // mm.shape[0], 0)
    if lens is not None:
        for i, n in enumerate(lens.tolist()):
            full[i, :, n:] = float("-inf")
    return full.numpy()


@pytest.mark.parametrize("decode_kernel", [True, False])
@pytest.mark.parametrize("bh,sq,sk,d,dtype,force,mask,kvl", CASES)
def test_pieces_match_oracle_and_plain_launch(bh, sq, sk, d, dtype, force, mask, kvl, decode_kernel, pieces):
    """Rows of one to four queries at head dim 64 / 128 run on the decode kernel (fp32 pieces), everything else --
    and everything with decode_kernel = False -- on the matrix-pipe kernels (pieces in the element type)."""
    if not decode_kernel and (sq > 4 or d not in (64, 128)):
        pytest.skip("not a decode-kernel shape: same route as with decode_kernel = True")
    q, k, v, m, lens = _inputs(bh, sq, sk, d, dtype, mask, kvl, seed=bh * 1000 + sk)
    tdt = q.dtype
    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    kw = dict(mask=None if m is None else m.to(tdt).cuda(), kv_len=None if lens is None else lens.cuda(), want_lse=True)
    pieces(force, decode_kernel)
    P = _params(bh, sq, sk, d, dtype=capi.F16 if dtype == "fp16" else capi.BF16)
    if m is not None:
        P.mask_kind, P.mask_bh_div, P.mask_stride_b, P.mask_stride_q = capi.MASK_ADDITIVE, bh // m.shape[0], sk, 0
    capi._sync_env()
    need = capi.lib().fmha_fwd_workspace_bytes(C.byref(P))
    assert need > 0, "the library would not run this launch in pieces"
    o, lse, _, _ = capi.fwd(qc, kc, vc, **kw)
    o0, lse0, _, _ = capi.fwd(qc, kc, vc, workspace=False, **kw)
    torch.cuda.synchronize()
    ref = oracle.attention(f32(q), f32(k), f32(v), mask=_oracle_mask(m if m is None else m.to(tdt), lens, bh, sq, sk),
                           want=("o", "lse"))
    assert np.abs(f32(o.cpu()) - ref["o"]).max() <= O_TOL[dtype]
    assert np.abs(f32(o0.cpu()) - ref["o"]).max() <= O_TOL[dtype]
    assert np.abs(lse.cpu().numpy() - ref["lse"]).max() <= 2e-3
    assert (o.float() - o0.float()).abs().max().item() <= SELF_TOL[dtype]
    assert (lse - lse0).abs().max().item() <= 5e-4


def test_run_time_layouts_and_too_small_workspaces(pieces):
    """K/V caches laid out [B, S, H, D] (a head's rows H*D apart) are cut the same way; a workspace that is
    too small, or none, gives the plain launch (bit-identical to workspace=False), never an error."""
    B, H, sq, sk, d = 2, 3, 1, 1300, 64
    g = torch.Generator().manual_seed(5)
    q = torch.randn(B, sq, H, d, generator=g).half().cuda().transpose(1, 2)
    k = torch.randn(B, sk, H, d, generator=g).half().cuda().transpose(1, 2)
    v = torch.randn(B, sk, H, d, generator=g).half().cuda().transpose(1, 2)
    lens = torch.tensor([1300, 517], dtype=torch.int32).cuda()
    pieces(4)
    o, lse, _, _ = capi.fwd(q, k, v, kv_len=lens, want_lse=True)
    o0, lse0, _, _ = capi.fwd(q, k, v, kv_len=lens, want_lse=True, workspace=False)
    tiny = torch.empty(64, dtype=torch.uint8, device="cuda")
    o1, _, _, _ = capi.fwd(q, k, v, kv_len=lens, workspace=tiny)
    big = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    o2, _, _, _ = capi.fwd(q, k, v, kv_len=lens, workspace=big)
    torch.cuda.synchronize()
    assert o.shape == o0.shape == (B, H, sq, d)
    assert torch.equal(o1, o0)
    assert torch.equal(o2, o) and big.any()  # the pieces did run: their partial results are in the workspace
    assert (o.float() - o0.float()).abs().max().item() <= SELF_TOL["fp16"]
    assert (lse - lse0).abs().max().item() <= 5e-4
    m = torch.zeros(B * H, sq, sk)
    for b, n in enumerate(lens.tolist()):
        m[b * H:(b + 1) * H, :, n:] = float("-inf")
    fold = lambda t: t.reshape(B * H, t.shape[2], d).cpu()
    ref = oracle.attention(f32(fold(q)), f32(fold(k)), f32(fold(v)), mask=m.numpy(), want=("o",))
    assert np.abs(f32(fold(o)) - ref["o"]).max() <= O_TOL["fp16"]


def test_launches_that_stay_whole(pieces):
    """Causal masks, dropout, mask tensors along the queries, many heads and short key ranges are not cut."""
    pieces(None)
    capi._sync_env()
    L = capi.lib()
    ok = _params(4, 1, 4096, 64)
    assert L.fmha_fwd_workspace_bytes(C.byref(ok)) > 0
    for kw in (dict(causal=1), dict(drop_kind=capi.DROP_PHILOX, p_drop=0.1),
               dict(mask_kind=capi.MASK_ADDITIVE, mask_bh_div=1, mask_stride_b=2 * 4096, mask_stride_q=4096, nq=2)):
        P = _params(4, kw.pop("nq", 1), 4096, 64, **kw)
        assert L.fmha_fwd_workspace_bytes(C.byref(P)) == 0, kw
    assert L.fmha_fwd_workspace_bytes(C.byref(_params(4096, 1, 4096, 64))) == 0   # enough heads to fill the chip
    assert L.fmha_fwd_workspace_bytes(C.byref(_params(4, 1, 512, 64))) == 0       # nothing to cut
    pieces(0)
    capi._sync_env()
    assert L.fmha_fwd_workspace_bytes(C.byref(ok)) == 0


def test_head_without_visible_keys_in_pieces(pieces):
    """A count of zero keys: O = 0 and LSE = -inf, as the plain launch gives."""
    bh, sk, d = 2, 600, 64
    q, k, v = (t.cuda() for t in make_qkv(bh, 1, sk, d, seed=1))
    lens = torch.tensor([0, 300], dtype=torch.int32).cuda()
    pieces(3)
    o, lse, _, _ = capi.fwd(q, k, v, kv_len=lens, want_lse=True)
    torch.cuda.synchronize()
    assert not o[0].any() and torch.isinf(lse[0]).all() and (lse[0] < 0).all()
    assert torch.isfinite(o[1].float()).all() and torch.isfinite(lse[1]).all()


def test_operator_allocates_the_workspace_itself():
    """torch.ops.mha_manual.fmha_fwd on a decode step: the pieces run (the result differs from the plain launch
    in the last place somewhere) and agree with it; the backward works from the merged LSE."""
    from nvfuserexamples_amd import load_ops
    ops = load_ops()
    bh, sk, d = 8, 4096, 64
    q, k, v = (t.cuda() for t in make_qkv(bh, 1, sk, d, seed=2))
    o, lse = ops.fmha_fwd(q, k, v, None, 0.0, False, 0.0, 0, 0, None)
    o0, lse0, _, _ = capi.fwd(q, k, v, want_lse=True, workspace=False)
    torch.cuda.synchronize()
    assert (o.float() - o0.float()).abs().max().item() <= SELF_TOL["fp16"]
    assert (lse - lse0).abs().max().item() <= 5e-4
    qg, kg, vg = (t.clone().requires_grad_(True) for t in (q, k, v))
    og = ops.fmha_fwd(qg, kg, vg, None, 0.0, False, 0.0, 0, 0, None)[0]
    do = torch.randn_like(og)
    og.backward(do)
    dq0, dk0, dv0 = capi.bwd(do, q, k, v, o0, lse0)
    torch.cuda.synchronize()
    for a, b in ((qg.grad, dq0), (kg.grad, dk0), (vg.grad, dv0)):
        assert (a.float() - b.float()).abs().max().item() <= 2e-3 * max(1.0, b.float().abs().max().item())


@pytest.mark.parametrize("d", [64, 200])
def test_ragged_last_piece_reads_no_row_past_the_end(d, pieces):
    """The last piece of the last head has fewer rows than the others (300 keys = 256 + 44): K and V sit at the
    end of buffers whose tails hold NaN, so a row read past the 300th would poison the output (head dim 200
    runs on the plain forward loop, 64 on the pipelined one)."""
    bh, sq, sk = 4, 129, 300
    q, k, v = make_qkv(bh, sq, sk, d, seed=17, std=STD[d])
    bufs = []
    for t in (k, v):
        buf = torch.full((bh * sk + 1024, d), float("nan"), dtype=torch.float16, device="cuda")
        buf[:bh * sk] = t.reshape(bh * sk, d).cuda()
        bufs.append(buf)
    kc, vc = (b[:bh * sk].view(bh, sk, d) for b in bufs)
    pieces(2)
    o, lse, _, _ = capi.fwd(q.cuda(), kc, vc, want_lse=True)
    torch.cuda.synchronize()
    ref = oracle.attention(f32(q), f32(k), f32(v), want=("o", "lse"))
    assert torch.isfinite(o.float()).all() and torch.isfinite(lse).all()
    assert np.abs(f32(o.cpu()) - ref["o"]).max() <= O_TOL["fp16"]


def test_randomized_decode_steps_against_the_oracle(monkeypatch):
    """150 seeded random problems of one to eight query rows (up to four: the decode kernel; e4m3 rows: up to four), head dim 64 / 128, fp16 / bf16 / e4m3 inputs,
    ragged key ranges, per-key masks (batch- or head-wise, with holes and -inf), valid key counts, folded and
    [B, S, H, D] layouts, whole key range or 2-7 pieces.  O within 2e-3 (fp16, e4m3 inputs) / 2e-2 (bf16) of the
    oracle, LSE within 2e-3, -inf rows in the same places."""
    import random
    rng = random.Random(424242)
    L = capi.lib()
    try:
        for it in range(150):
            kind = rng.choice(["fp16", "fp16", "bf16", "e4m3"])
            d = rng.choice([64, 128])
            b, h = rng.choice([1, 2, 3]), rng.choice([1, 2, 4])
            bh = b * h
            sq = rng.choice([1, 1, 1, 2, 3, 4]) if kind == "e4m3" else rng.choice([1, 1, 1, 2, 3, 4, 5, 8])
            sk = rng.choice([1, 7, 33, 64, 100, 255, 256, 257, 500, 1000, 1777, 3000])
            maskk = rng.choice(["none", "none", "pad", "head"])
            use_len = rng.random() < 0.4
            strided = kind != "e4m3" and rng.random() < 0.3
            n = rng.choice([0, 0, 2, 3, 7])
            g = torch.Generator().manual_seed(1000 + it)
            std = 1.0 if d == 64 else 0.5
            tdt = torch.bfloat16 if kind == "bf16" else torch.float16
            q, k, v = (torch.randn(bh, s, d, generator=g) * std for s in (sq, sk, sk))
            m = None
            if maskk == "pad":
                m = torch.zeros(b, 1, 1, sk)
                for i in range(b):
                    m[i, ..., rng.randint(1, sk):] = -10000.0
            elif maskk == "head":
                m = torch.randn(bh, 1, sk, generator=g)
                m[torch.rand(bh, 1, sk, generator=g) < 0.3] = float("-inf")
            lens = torch.tensor([rng.randint(0, sk) for _ in range(b)], dtype=torch.int32) if use_len else None
            monkeypatch.setenv("FMHA_FWD_SPLIT", str(n))
            mc = None if m is None else m.to(tdt).cuda()
            lc = None if lens is None else lens.cuda()
            if kind == "e4m3":
                q8, k8, v8 = (t.to(torch.float8_e4m3fn) for t in (q, k, v))
                o, lse = capi.fwd_fp8(q8.cuda(), k8.cuda(), v8.cuda(), 0.5, 2.0, 0.25, mask=mc, out_dtype=tdt,
                                      want_lse=True, kv_len=lc)
                qf, kf, vf, scale = f32(q8.float()), f32(k8.float()), f32(v8.float()) * np.float32(0.25), d ** -0.5
            else:
                qc, kc, vc = (t.to(tdt).cuda() for t in (q, k, v))
                if strided:
                    lay = lambda x: x.view(b, h, x.shape[1], d).permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
                    qc, kc, vc = lay(qc), lay(kc), lay(vc)
                o, lse, _, _ = capi.fwd(qc, kc, vc, mask=mc, want_lse=True, kv_len=lc)
                qf, kf, vf, scale = f32(q.to(tdt)), f32(k.to(tdt)), f32(v.to(tdt)), d ** -0.5
            torch.cuda.synchronize()
            full = np.zeros((bh, sq, sk), np.float32)
            if m is not None:
                mm = f32(m.to(tdt)).reshape(-1, 1, sk)
                full += np.repeat(mm, bh // mm.shape[0], 0)
            if lens is not None:
                for i, cnt in enumerate(lens.tolist()):
                    full[i * h:(i + 1) * h, :, cnt:] = -np.inf
            ref = oracle.attention(qf, kf, vf, mask=full, scale=scale, want=("o", "lse"))
            what = f"case #{it}: {kind} d{d} b{b} h{h} sq{sq} sk{sk} mask {maskk} len {use_len} strided {strided} pieces {n}"
            tol = (2e-2 if kind == "bf16" else 2e-3) * max(1.0, float(np.abs(ref["o"]).max()) / 2.0)
            assert np.abs(f32(o.reshape(bh, sq, d).cpu()) - ref["o"]).max() <= tol, what
            fin = np.isfinite(ref["lse"])
            gl = lse.reshape(bh, sq).cpu().numpy()
            assert np.array_equal(np.isfinite(gl), fin), what
            assert not fin.any() or np.abs(gl[fin] - ref["lse"][fin]).max() <= 2e-3 + 2.0 ** -8 * (kind == "bf16"), what
    finally:
        monkeypatch.delenv("FMHA_FWD_SPLIT", raising=False)
        L.fmha_reload_overrides()
