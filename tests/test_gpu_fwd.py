"""GPU parity of the forward path, called through the C ABI (ctypes -> libfmha_hip.so).

Bars (fp16): max |O - oracle| <= 2e-3 against the unrounded fp64-accumulated oracle of the
eager composition (reference test.py:12-18); bf16 is held to 2e-2 (8-bit mantissa: the
probabilities and the output each carry 2^-9 relative rounding).  The reference itself
asserts atol=1e-2 (test.py:29).  Dropout keep decisions are bit-exact.
"""
import numpy as np
import pytest
import torch

import oracle
from nvfuserexamples_amd import capi
from conftest import make_qkv, pad_mask, tail_mask, f32

pytestmark = pytest.mark.gpu

TOL = {"fp16": 2e-3, "bf16": 2e-2}
# The kernel's softmax denominator sums the probabilities AFTER rounding to the element type (so the
# weights of the second product sum to one exactly); the saved LSE carries that rounding: up to
# 2^-11 relative (fp16) / 2^-9 (bf16) on rows with a handful of visible keys.
LSE_TOL = {"fp16": 1e-3, "bf16": 5e-3}
# Q is pre-multiplied by scale * log2(e) and rounded ONCE to the element type before the first
# product, so every score carries that rounding (2^-11 / 2^-8 relative).  A row with one or two
# visible keys shows it in full in its LSE, hence the term proportional to |LSE| where such rows occur.
LSE_REL = {"fp16": 2.0 ** -11, "bf16": 2.0 ** -8}
TDT = {"fp16": torch.float16, "bf16": torch.bfloat16}


def _run(q, k, v, **kw):
    out = capi.fwd(q.cuda(), k.cuda(), v.cuda(), **kw)
    torch.cuda.synchronize()
    return out


CASES = [
    # bh, sq, sk, d, dtype, mask, causal
    (4, 128, 128, 64, "fp16", None, False),
    (4, 128, 128, 64, "fp16", "keep01", False),       # the reference's inference op layout
    (6, 128, 128, 64, "fp16", "pad", False),          # [B,1,1,S] padding mask, B = 3
    (4, 512, 512, 64, "fp16", "pad", False),          # headline sequence length
    (2, 512, 512, 64, "fp16", "add_full", False),
    (3, 100, 77, 64, "fp16", None, False),            # ragged
    (2, 1, 1, 64, "fp16", None, False),               # one query, one key
    (2, 33, 257, 64, "fp16", "add_full", False),      # ragged, mask rows not 8-byte aligned
    (2, 320, 320, 64, "fp16", None, True),            # causal
    (2, 200, 200, 64, "fp16", "pad", True),           # causal + padding
    (2, 2048, 2048, 64, "fp16", None, False),         # long sequence: many K/V tiles
    (2, 256, 256, 128, "fp16", None, False),
    (2, 1024, 1024, 128, "bf16", None, True),         # wide-head bf16 causal
    (4, 192, 192, 64, "bf16", "pad", False),
    # head dim 256 (built for coverage: plain loop, one wave per SIMD)
    (2, 256, 256, 256, "fp16", None, False),
    (2, 200, 333, 256, "fp16", "pad", False),
    (2, 130, 257, 256, "fp16", "add_full", False),
    (2, 320, 320, 256, "bf16", None, True),
    (3, 100, 77, 256, "bf16", "pad", True),
    (2, 192, 192, 256, "fp16", "pad", True),
]


@pytest.mark.parametrize("qb", [1, 2])
@pytest.mark.parametrize("bh,sq,sk,d,dtype,mask,causal", CASES)
def test_forward_matches_oracle(bh, sq, sk, d, dtype, mask, causal, qb, monkeypatch):
    monkeypatch.setenv("FMHA_FWD_QB", str(qb))
    std = {64: 1.0, 128: 0.5, 256: 0.35}[d]
    q, k, v = make_qkv(bh, sq, sk, d, seed=bh + sq, std=std, dtype=dtype)
    m, mk = None, capi.MASK_ADDITIVE
    g = torch.Generator().manual_seed(sq)
    if mask == "pad":
        m = pad_mask(bh // 2, sk, sk // 2, sk)
    elif mask == "keep01":
        m, mk = torch.empty(bh, sq, sk).random_(2, generator=g), capi.MASK_KEEP01
    elif mask == "add_full":
        m = torch.randn(bh, sq, sk, generator=g) * 2
    if m is not None:
        m = m.to(TDT[dtype])
    o, lse, _, _ = _run(q, k, v, mask=None if m is None else m.cuda(), mask_kind=mk, causal=causal, want_lse=True)
    ref = oracle.attention(f32(q), f32(k), f32(v), mask=None if m is None else f32(m),
                           mask_kind="keep01" if mk == capi.MASK_KEEP01 else "additive", causal=causal,
                           want=("o", "lse"))
    assert np.abs(f32(o.cpu()) - ref["o"]).max() <= TOL[dtype]
    assert np.abs(lse.cpu().numpy() - ref["lse"]).max() <= LSE_TOL[dtype]


# The forward kernel is persistent: the grid is capped at the number of workgroups the device
# keeps resident (two per CU: 512 on a 256-CU part) and each workgroup walks several (head,
# query tile) items, prefetching the next item's Q rows and first K tiles while it works.
# These shapes have more items than any such grid, few key tiles per item (so the prefetch
# stream crosses item boundaries every other tile, and with two tiles per item reaches the
# item after next), and masks that differ from head to head.
MANY_ITEMS = [
    # bh, sq, sk, d, dtype, mask, causal, qb
    (600, 128, 128, 64, "fp16", "pad", False, 1),    # 600 items of two key tiles
    (600, 128, 100, 64, "fp16", "pad", False, 1),    # ... of one key tile and a phantom tile
    (560, 192, 192, 64, "fp16", "pad", True, 1),     # causal: 1120 items of unequal length
    (520, 128, 200, 128, "bf16", None, False, 1),    # head dim 128: Q comes from global memory per item
    (1040, 256, 64, 64, "fp16", "pad", False, 2),    # two query blocks per wave: 32-key tiles, 1040 items
    (1040, 256, 200, 64, "fp16", None, False, 2),
]


@pytest.mark.parametrize("bh,sq,sk,d,dtype,mask,causal,qb", MANY_ITEMS)
def test_forward_many_items_per_workgroup(bh, sq, sk, d, dtype, mask, causal, qb, monkeypatch):
    monkeypatch.setenv("FMHA_FWD_QB", str(qb))
    q, k, v = make_qkv(bh, sq, sk, d, seed=bh + sk, std=0.5 if d == 128 else 1.0, dtype=dtype)
    m = None
    if mask == "pad":
        m = pad_mask(bh // 2, sk, 1, sk).to(TDT[dtype])  # one row per pair of heads, valid lengths in [1, sk]
    o, lse, _, _ = _run(q, k, v, mask=None if m is None else m.cuda(), causal=causal, want_lse=True)
    ref = oracle.attention(f32(q), f32(k), f32(v), mask=None if m is None else f32(m), causal=causal,
                           want=("o", "lse"))
    assert np.abs(f32(o.cpu()) - ref["o"]).max() <= TOL[dtype]
    assert (np.abs(lse.cpu().numpy() - ref["lse"]) <= LSE_TOL[dtype] + LSE_REL[dtype] * np.abs(ref["lse"])).all()


@pytest.mark.parametrize("bh,sq,sk,d,causal", [(3, 128, 192, 64, False), (2, 257, 257, 64, True),
                                                (2, 128, 128, 128, False)])
def test_philox_dropout_forward_and_mask_bit_exact(bh, sq, sk, d, causal):
    q, k, v = make_qkv(bh, sq, sk, d, seed=3)
    seed, offset, p = 0xfeedbeefcafe, (1 << 33) + 5, 0.1
    o, lse, _, _ = _run(q, k, v, causal=causal, drop_kind=capi.DROP_PHILOX, p_drop=p, seed=seed, offset=offset,
                        want_lse=True)
    ref = oracle.attention(f32(q), f32(k), f32(v), causal=causal, philox=True, p_drop=p,
                           seed=seed, offset=offset, want=("o", "lse"))
    assert np.abs(f32(o.cpu()) - ref["o"]).max() <= 2e-3
    assert np.abs(lse.cpu().numpy() - ref["lse"]).max() <= 1e-3
    # the keep decisions themselves: GPU materialisation == CPU rule, bit for bit
    km = capi.philox_keep_mask(seed, offset, p, bh, sq, sk).cpu().numpy()
    assert np.array_equal(km, oracle.keep_mask(seed, offset, p, bh, sq, sk))
    # and the fused kernel used exactly those decisions: feeding them back as an explicit
    # dropout tensor reproduces its output to rounding
    o2, _, _, _ = _run(q, k, v, drop_kind=capi.DROP_TENSOR, drop_mask=torch.from_numpy(km).to(q.dtype).cuda(),
                       drop_scale=capi.lib().fmha_drop_scale(p)) if not causal else (o, None, None, None)
    assert np.abs(f32(o2.cpu()) - f32(o.cpu())).max() <= 1e-3


def test_train_ops_and_saved_intermediates():
    """Reference train semantics (test_train_mha.py:14-21) incl. the saved softmax / dropout tensors;
    the zero pattern of the dropped output is the caller's mask, exactly."""
    bh, s, d = 8, 128, 64
    q, k, v = make_qkv(bh, s, s, d, seed=8)
    g = torch.Generator().manual_seed(2)
    pm = (torch.empty(bh, s, s).random_(2, generator=g) * -1000).half()
    dm = torch.empty(bh, s, s).random_(2, generator=g).half()
    o, _, sm, dr = _run(q, k, v, mask=pm.cuda(), drop_kind=capi.DROP_TENSOR, drop_mask=dm.cuda(), drop_scale=2.0,
                        save=True)
    ref = oracle.attention(f32(q), f32(k), f32(v), mask=f32(pm), drop_mask=f32(dm), drop_scale=2.0,
                           want=("o", "softmax", "dropout"))
    assert np.abs(f32(o.cpu()) - ref["o"]).max() <= 4e-3   # O is up to 2x larger here (x2 scaling)
    assert np.abs(f32(sm.cpu()) - ref["softmax"]).max() <= 1e-3
    assert np.abs(f32(dr.cpu()) - ref["dropout"]).max() <= 2e-3
    live = ref["softmax"] > 1e-6
    assert np.array_equal((f32(dr.cpu()) == 0)[live], (f32(dm) == 0)[live])
    o2, _, _, _ = _run(q, k, v, mask=pm.cuda(), drop_kind=capi.DROP_TENSOR, drop_mask=dm.cuda(), drop_scale=2.0)
    assert torch.equal(o2, o)  # the save pass does not disturb O


# Key ranges of at most 128 keys under a full mask tensor whose rows start on 16-byte boundaries run on a
# one-pass kernel of their own (exact row maximum, whole-row accesses to the [.., sq, sk] tensors): the
# reference's three operators at their own shape.  FMHA_FWD_SHORT=0 keeps the same calls on the general
# kernels; both must meet the oracle.
SHORT = [
    # bh, sq, sk, dtype, mode
    (4, 128, 128, "fp16", "infer"),     # the reference's inference operator (0/1 mask -> (1-m) * -10000)
    (4, 128, 40, "fp16", "infer"),      # one partly filled key block
    (6, 33, 64, "fp16", "train"),       # ragged query rows, dropout tensor
    (5, 200, 96, "fp16", "save"),       # two query tiles, three key blocks
    (3, 77, 8, "fp16", "save"),         # a single 16-byte chunk per row
    (4, 300, 128, "bf16", "save"),
    (600, 128, 128, "fp16", "train"),   # more workgroups than the device holds at once
    (6, 160, 128, "fp16", "bcast"),     # [B,1,sq,sk] mask shared by the heads of a batch entry, -inf entries, LSE
    # beyond 128 keys the same operators run on a streaming kernel (whole-row accesses, online softmax over
    # 64-key tiles); FMHA_FWD_STREAM=0 keeps them on the pipelined kernel
    (4, 512, 512, "fp16", "infer"),
    (3, 200, 264, "fp16", "train"),     # ragged query tile, partly filled last key tile
    (4, 128, 320, "bf16", "train"),
    (2, 33, 1024, "fp16", "infer"),     # sixteen key tiles
    (300, 128, 192, "fp16", "train"),   # more workgroups than the device holds at once
    (6, 160, 256, "fp16", "bcast"),
    (3, 100, 136, "fp16", "save"),      # saved outputs from the streaming forward's LSE
]


@pytest.mark.parametrize("short", ["1", "0"])
@pytest.mark.parametrize("bh,sq,sk,dtype,mode", SHORT)
def test_short_key_ranges_under_full_masks(bh, sq, sk, dtype, mode, short, monkeypatch):
    monkeypatch.setenv("FMHA_FWD_SHORT", short)
    monkeypatch.setenv("FMHA_FWD_STREAM", short)
    q, k, v = make_qkv(bh, sq, sk, 64, seed=bh + sk, dtype=dtype)
    g = torch.Generator().manual_seed(sq + sk)
    tol = TOL[dtype]
    if mode == "infer":
        m = torch.empty(bh, sq, sk).random_(2, generator=g).to(TDT[dtype])
        o, lse, _, _ = _run(q, k, v, mask=m.cuda(), mask_kind=capi.MASK_KEEP01, want_lse=True)
        ref = oracle.attention(f32(q), f32(k), f32(v), mask=f32(m), mask_kind="keep01", want=("o", "lse"))
        assert np.abs(f32(o.cpu()) - ref["o"]).max() <= tol
        assert np.abs(lse.cpu().numpy() - ref["lse"]).max() <= LSE_TOL[dtype]
        return
    if mode == "bcast":
        m = torch.randn(bh // 3, 1, sq, sk, generator=g) * 2
        m[:, :, :, 5::7] = float("-inf")
        m[0, 0, 3, :] = float("-inf")          # a query that sees no key at all: O = 0, LSE = -inf
        m = m.to(TDT[dtype])
        o, lse, _, _ = _run(q, k, v, mask=m.cuda(), want_lse=True)
        ref = oracle.attention(f32(q), f32(k), f32(v), mask=f32(m), want=("o", "lse"))
        assert np.abs(f32(o.cpu()) - ref["o"]).max() <= tol
        got = lse.cpu().numpy()
        dead = np.isneginf(ref["lse"])
        assert dead.any() and np.array_equal(np.isneginf(got), dead)
        assert np.abs(got[~dead] - ref["lse"][~dead]).max() <= LSE_TOL[dtype]
        assert (f32(o.cpu())[dead] == 0).all()
        return
    pm = (torch.empty(bh, sq, sk).random_(2, generator=g) * -1000).to(TDT[dtype])
    dm = torch.empty(bh, sq, sk).random_(2, generator=g).to(TDT[dtype])
    o, _, sm, dr = _run(q, k, v, mask=pm.cuda(), drop_kind=capi.DROP_TENSOR, drop_mask=dm.cuda(), drop_scale=2.0,
                        save=(mode == "save"))
    ref = oracle.attention(f32(q), f32(k), f32(v), mask=f32(pm), drop_mask=f32(dm), drop_scale=2.0,
                           want=("o", "softmax", "dropout"))
    assert np.abs(f32(o.cpu()) - ref["o"]).max() <= 2 * tol   # O is up to 2x larger here (x2 scaling)
    if mode == "save":
        assert np.abs(f32(sm.cpu()) - ref["softmax"]).max() <= tol / 2
        assert np.abs(f32(dr.cpu()) - ref["dropout"]).max() <= tol
        live = ref["softmax"] > 1e-6
        assert np.array_equal((f32(dr.cpu()) == 0)[live], (f32(dm) == 0)[live])
        o2, _, _, _ = _run(q, k, v, mask=pm.cuda(), drop_kind=capi.DROP_TENSOR, drop_mask=dm.cuda(), drop_scale=2.0)
        assert torch.equal(o2, o)  # saving does not disturb O


# Beyond 128 keys the saved outputs come, up to 512 keys, from one launch that keeps a wave's probabilities in
# registers until the row's log-sum-exp is known; FMHA_FWD_SAVE_ONCE=0 (and any longer key range): from a streaming
# kernel that follows the forward launch and derives them from its row log-sum-exp; FMHA_FWD_SAVE_SPLIT=0 as well:
# from a second sweep inside a plain forward kernel, which is also what serves rows that do not start on 16-byte
# boundaries and head dim 128.
SAVE_LONG = [
    # bh, sq, sk, d, dtype
    (6, 200, 264, 64, "fp16"),     # ragged query tiles, a partly filled last key tile
    (3, 128, 512, 64, "fp16"),
    (4, 192, 320, 64, "bf16"),
    (300, 128, 192, 64, "fp16"),   # more workgroups than the device holds at once
    (3, 100, 333, 64, "fp16"),     # rows not 16-byte aligned: the plain kernel either way
    (2, 160, 256, 128, "fp16"),    # head dim 128: the plain kernel either way
]


@pytest.mark.parametrize("route", ["once", "split", "plain"])
@pytest.mark.parametrize("bh,sq,sk,d,dtype", SAVE_LONG)
def test_saved_intermediates_beyond_128_keys(bh, sq, sk, d, dtype, route, monkeypatch):
    split = "0" if route == "plain" else "1"
    monkeypatch.setenv("FMHA_FWD_SAVE_ONCE", "1" if route == "once" else "0")
    monkeypatch.setenv("FMHA_FWD_SAVE_SPLIT", split)
    # without the split the saving forward is the plain kernel, whose O is bit-identical to the pipelined
    # kernel's, not to the streaming kernel's: keep the non-saving call on the same family
    monkeypatch.setenv("FMHA_FWD_STREAM", split)
    q, k, v = make_qkv(bh, sq, sk, d, seed=bh + sk, std=0.5 if d == 128 else 1.0, dtype=dtype)
    g = torch.Generator().manual_seed(sq + sk)
    pm = (torch.empty(bh, sq, sk).random_(2, generator=g) * -1000).to(TDT[dtype])
    dm = torch.empty(bh, sq, sk).random_(2, generator=g).to(TDT[dtype])
    o, _, sm, dr = _run(q, k, v, mask=pm.cuda(), drop_kind=capi.DROP_TENSOR, drop_mask=dm.cuda(), drop_scale=2.0,
                        save=True)
    ref = oracle.attention(f32(q), f32(k), f32(v), mask=f32(pm), drop_mask=f32(dm), drop_scale=2.0,
                           want=("o", "softmax", "dropout"))
    tol = TOL[dtype]
    assert np.abs(f32(o.cpu()) - ref["o"]).max() <= 2 * tol
    assert np.abs(f32(sm.cpu()) - ref["softmax"]).max() <= tol / 2
    assert np.abs(f32(dr.cpu()) - ref["dropout"]).max() <= tol
    live = ref["softmax"] > 1e-6
    assert np.array_equal((f32(dr.cpu()) == 0)[live], (f32(dm) == 0)[live])
    o2, _, _, _ = _run(q, k, v, mask=pm.cuda(), drop_kind=capi.DROP_TENSOR, drop_mask=dm.cuda(), drop_scale=2.0)
    assert torch.equal(o2, o)  # saving does not disturb O


@pytest.mark.parametrize("route", ["once", "split"])
def test_saved_intermediates_of_rows_that_meet_their_first_key_late_or_never(route, monkeypatch):
    """The one-launch kernel rescales a tile's kept probabilities by exp2(m_t - L): rows that see no key at all
    (L = -inf), rows whose first tiles are entirely -inf (m_t = -inf there), and rows whose early keys carry a
    finite -10000 while later ones carry 0 (m_t far below L: the factor underflows to zero, as the true value does)."""
    monkeypatch.setenv("FMHA_FWD_SAVE_ONCE", "1" if route == "once" else "0")
    bh, sq, sk = 3, 160, 448
    q, k, v = make_qkv(bh, sq, sk, 64, seed=77)
    g = torch.Generator().manual_seed(78)
    pm = torch.randn(bh, sq, sk, generator=g)
    pm[:, 5, :] = float("-inf")                 # never a key
    pm[:, 9, :200] = float("-inf")              # three whole tiles and part of the fourth before the first key
    pm[:, 17, :320] = -10000.0                  # finite but hopeless early keys
    pm[:, 33, 64:] = float("-inf")              # only the first tile counts
    pm[1, :, 128:192] = float("-inf")           # a whole tile dead for every row of a head
    pm = pm.half()
    dm = torch.empty(bh, sq, sk).random_(2, generator=g).half()
    o, lse, sm, dr = _run(q, k, v, mask=pm.cuda(), drop_kind=capi.DROP_TENSOR, drop_mask=dm.cuda(), drop_scale=1.25,
                          save=True, want_lse=True)
    ref = oracle.attention(f32(q), f32(k), f32(v), mask=f32(pm), drop_mask=f32(dm), drop_scale=1.25,
                           want=("o", "lse", "softmax", "dropout"))
    tol = TOL["fp16"]
    got_sm, got_dr = f32(sm.cpu()), f32(dr.cpu())
    assert np.isfinite(got_sm).all() and np.isfinite(got_dr).all() and np.isfinite(f32(o.cpu())).all()
    assert np.abs(f32(o.cpu()) - ref["o"]).max() <= 2 * tol
    assert np.abs(got_sm - ref["softmax"]).max() <= tol / 2
    assert np.abs(got_dr - ref["dropout"]).max() <= tol
    assert (got_sm[:, 5] == 0).all() and (got_dr[:, 5] == 0).all() and (f32(o.cpu())[:, 5] == 0).all()
    assert (got_sm[:, 9, :200] == 0).all() and (got_sm[:, 17, :320] == 0).all() and (got_sm[1, :, 128:192] == 0).all()
    gl = lse.cpu().numpy()
    dead = np.isneginf(ref["lse"])
    assert dead.any() and np.array_equal(np.isneginf(gl), dead)
    assert np.abs(gl[~dead] - ref["lse"][~dead]).max() <= LSE_TOL["fp16"]


@pytest.mark.parametrize("bh,sq,sk,d,dtype,mask", [
    (6, 200, 333, 64, "fp16", "pad"),        # ragged tiles, per-key mask
    (4, 192, 192, 64, "bf16", "add_full"),   # full mask tensor and dropout tensor together
    (600, 128, 192, 64, "fp16", None),       # more items than resident workgroups
    (4, 160, 224, 128, "fp16", "pad"),       # head dim 128: the plain kernel
])
def test_tensor_dropout_matches_oracle(bh, sq, sk, d, dtype, mask):
    """An explicit 0/1 dropout tensor scaled by 2 (reference fmha/fmha_manual.cpp:478-480) beyond the
    reference's fixed shape: ragged tiles, broadcast and full masks, many items per workgroup."""
    q, k, v = make_qkv(bh, sq, sk, d, seed=bh + sq, std=0.5 if d == 128 else 1.0, dtype=dtype)
    g = torch.Generator().manual_seed(sk)
    dm = torch.empty(bh, sq, sk).random_(2, generator=g).to(TDT[dtype])
    m = None
    if mask == "pad":
        m = pad_mask(2, sk, sk // 2, sk).to(TDT[dtype])
    elif mask == "add_full":
        m = (torch.empty(bh, sq, sk).random_(2, generator=g) * -1000).to(TDT[dtype])
    o, _, _, _ = _run(q, k, v, mask=None if m is None else m.cuda(), drop_kind=capi.DROP_TENSOR, drop_mask=dm.cuda(),
                      drop_scale=2.0)
    ref = oracle.attention(f32(q), f32(k), f32(v), mask=None if m is None else f32(m), drop_mask=f32(dm),
                           drop_scale=2.0, want=("o",))
    assert np.abs(f32(o.cpu()) - ref["o"]).max() <= (4e-3 if dtype == "fp16" else 4e-2)   # O is up to 2x larger here


@pytest.mark.parametrize("d,dtype", [(128, "fp16"), (128, "bf16"), (256, "fp16"), (256, "bf16")])
@pytest.mark.parametrize("kind", ["first_tile", "first_key", "all", "all_but_last"])
def test_plain_loop_under_masks_that_hide_the_first_keys(kind, d, dtype):
    """The plain (not pipelined) forward loop -- tensor dropout at head dim 128, everything at head dim
    256 -- sets its reference exponent at the first tile that has a finite score.  Under a -10000 mask
    that first reference lies thousands below zero and the next one thousands above it; neither move may
    touch the (still empty) sums.  A fully masked row is a plain softmax (reference fmha/fmha_manual.cpp:70)."""
    bh, sq, sk = 4, 100, 200
    q, k, v = make_qkv(bh, sq, sk, d, seed=d + sk, std=0.5 if d == 128 else 0.35, dtype=dtype)
    m = torch.zeros(2, 1, 1, sk)
    if kind == "first_tile":
        m[..., :64] = -10000.0
    elif kind == "first_key":
        m[..., 0] = -10000.0
    elif kind == "all":
        m[0] = -10000.0
    elif kind == "all_but_last":
        m[..., : sk - 1] = -10000.0
    m = m.to(TDT[dtype])
    kw, okw = {}, {}
    if d == 128:  # the dropout tensor (all ones) is what selects the plain loop at this head dim
        dm = torch.ones(bh, sq, sk).to(TDT[dtype])
        kw, okw = dict(drop_kind=capi.DROP_TENSOR, drop_mask=dm.cuda(), drop_scale=1.0), dict(drop_mask=f32(dm), drop_scale=1.0)
    o = _run(q, k, v, mask=m.cuda(), **kw)[0]
    ref = oracle.attention(f32(q), f32(k), f32(v), mask=f32(m), want=("o",), **okw)
    assert not torch.isnan(o).any()
    assert np.abs(f32(o.cpu()) - ref["o"]).max() <= TOL[dtype]


def test_a_caller_built_against_an_older_header_keeps_working():
    """The parameter struct carries its own size: the library reads that many bytes and takes the fields
    beyond them as zero, whatever the memory after a shorter struct holds."""
    import ctypes as C
    q, k, v = (t.cuda() for t in make_qkv(4, 96, 160, 64, seed=6))
    want = capi.fwd(q, k, v)[0]
    P = capi.FwdParams()
    o = torch.empty_like(q)
    P.q, P.k, P.v, P.o = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr()
    P.bh, P.sq, P.sk, P.d = 4, 96, 160, 64
    P.dtype, P.scale = capi.F16, 64 ** -0.5
    # everything from kv_len on is "after the end" of an old caller's struct: poison it
    P.struct_bytes = capi.FwdParams.kv_len.offset
    P.kv_len, P.kv_len_bh_div, P.heads = 0xdead0, 3, 5
    P.q_stride[:] = [7, 7, 7]
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert capi.lib().fmha_fwd_launch(C.byref(P), stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(o, want)


def test_size_independent_properties_at_headline_shape():
    """B32 H16 S512 D64 (full size): properties that need no CPU answer, plus oracle parity on a
    sample of heads."""
    B, H, S, D = 32, 16, 512, 64
    q, k, v = make_qkv(B * H, S, S, D, seed=0)
    m = pad_mask(B, S, S // 2, S).half()
    qc, kc, vc, mc = q.cuda(), k.cuda(), v.cuda(), m.cuda()
    o = capi.fwd(qc, kc, vc, mask=mc)[0]
    # permuting the keys (K, V and the mask together) leaves O unchanged up to rounding
    perm = torch.randperm(S, generator=torch.Generator().manual_seed(1)).cuda()
    o_p = capi.fwd(qc, kc[:, perm].contiguous(), vc[:, perm].contiguous(), mask=mc[..., perm].contiguous())[0]
    assert (o_p.float() - o.float()).abs().max().item() <= 2e-3
    # linear in V
    v2 = make_qkv(B * H, S, S, D, seed=5)[2].cuda()
    o_a = capi.fwd(qc, kc, v2, mask=mc)[0]
    o_s = capi.fwd(qc, kc, (vc.float() + v2.float()).half(), mask=mc)[0]
    assert (o_s.float() - (o.float() + o_a.float())).abs().max().item() <= 6e-3
    # exact ones: V = 1 gives O = 1 (the weights are the rounded probabilities over THEIR sum), and doubling V
    # doubles O bit for bit (a power of two commutes with every rounding on the way, outside the subnormal range)
    o_1 = capi.fwd(qc, kc, torch.ones_like(vc), mask=mc)[0]
    assert torch.equal(o_1, torch.ones_like(o_1))
    o_2 = capi.fwd(qc, kc, vc * 2, mask=mc)[0]
    big = o.float().abs() >= 2.0 ** -13       # (a doubled value that leaves fp16's subnormal range carries bits its half had lost)
    assert torch.equal(o_2[big], (o * 2)[big])
    # masked keys carry no weight: scrambling V on the padded tail changes nothing
    lens = (m[:, 0, 0] == 0).sum(-1)
    v3 = vc.clone().view(B, H, S, D)
    for b in range(B):
        v3[b, :, lens[b]:] = 100.0
    o_t = capi.fwd(qc, kc, v3.view(B * H, S, D), mask=mc)[0]
    assert torch.equal(o_t, o)
    torch.cuda.synchronize()
    heads = [0, 17, 255, 511]
    ref = oracle.attention(f32(q[heads]), f32(k[heads]), f32(v[heads]),
                           mask=f32(m[[h // H for h in heads]]).reshape(len(heads), 1, S))["o"]
    assert np.abs(f32(o[heads].cpu()) - ref).max() <= 2e-3


def test_golden_fixture():
    """Committed seeded vectors (tests/golden/make_fixtures.py): inputs and oracle outputs."""
    import os
    f = np.load(os.path.join(os.path.dirname(__file__), "golden", "fwd_small.npz"))
    q, k, v, m = (torch.from_numpy(f[n]).half() for n in ("q", "k", "v", "mask"))
    o, lse, _, _ = _run(q, k, v, mask=m.cuda(), drop_kind=capi.DROP_PHILOX, p_drop=float(f["p_drop"]),
                        seed=int(f["seed"]), offset=int(f["offset"]), want_lse=True)
    assert np.abs(f32(o.cpu()) - f["o"]).max() <= 2e-3
    assert np.abs(lse.cpu().numpy() - f["lse"]).max() <= 1e-3


# A [B,1,1,sk] mask that ends in hard-masked keys (-10000 or -inf on the tail of every padded
# sequence) lets the pipelined forward skip the key tiles that hold nothing else.  The skipped
# keys' weights are exactly zero either way, so the result must equal, bit for bit, that of a
# launch which visits every tile (FLAG_NO_MASK_TRIM), and match the oracle like any other forward.
TRIM = [
    # bh, sq, sk, d, dtype, kind, causal, extra, heads per mask row
    (8, 512, 512, 64, "fp16", "tail", False, None, 2),
    (8, 512, 512, 64, "fp16", "inf", False, None, 2),
    (8, 512, 512, 64, "fp16", "holes", False, None, 2),
    (8, 512, 512, 64, "fp16", "soft", False, None, 2),
    (8, 256, 512, 64, "fp16", "last_live", False, None, 2),
    (8, 512, 512, 64, "fp16", "some_rows_all_masked", False, None, 2),
    (6, 300, 333, 64, "bf16", "tail", False, None, 2),          # ragged; -10000 is -9984 in bf16
    (4, 256, 1024, 64, "fp16", "tail", False, None, 2),         # the longest rows that are looked at
    (4, 128, 1100, 64, "fp16", "tail", False, None, 2),         # beyond: not looked at
    (4, 256, 320, 128, "bf16", "tail", False, None, 2),
    (4, 384, 384, 64, "fp16", "tail", True, None, 2),           # causal: both limits apply
    (8, 512, 512, 64, "fp16", "tail", False, "philox", 2),      # keep decisions depend on positions only
    (8, 512, 512, 64, "fp16", "holes", False, "kv_len", 2),     # valid key counts on top of the mask
    (600, 128, 256, 64, "fp16", "tail", False, None, 2),        # several items per workgroup
    (2400, 128, 256, 64, "fp16", "tail", False, None, 2),       # more than are looked at: no trimming
    # Shapes at which every workgroup of the persistent kernel has the same number of items (2 to 4)
    # and the mask has at most 64 rows: there all mask rows are looked at by every workgroup and dealt
    # to the workgroups by length, which changes which workgroup computes what but not the results.
    (512, 512, 512, 64, "fp16", "tail", False, None, 16),        # the headline shape
    (512, 512, 512, 64, "fp16", "holes", False, None, 16),
    (512, 512, 512, 64, "fp16", "some_rows_all_masked", False, None, 16),
    (512, 512, 512, 64, "fp16", "last_live", False, None, 16),
    (512, 512, 512, 64, "fp16", "tail", False, "philox", 16),
    (256, 512, 512, 64, "bf16", "tail", False, None, 16),        # two items per workgroup
    (256, 1024, 1024, 64, "fp16", "tail", False, None, 16),      # rows of two 512-key halves
    (384, 512, 520, 64, "fp16", "tail", False, None, 16),        # three items per workgroup; 520 keys
    (512, 512, 512, 64, "fp16", "tail", False, None, 8),         # 64 mask rows
]


@pytest.mark.parametrize("qb", [1, 2])
@pytest.mark.parametrize("bh,sq,sk,d,dtype,kind,causal,extra,heads", TRIM)
def test_trailing_hard_masked_keys_are_skipped_exactly(bh, sq, sk, d, dtype, kind, causal, extra, heads, qb, monkeypatch):
    monkeypatch.setenv("FMHA_FWD_QB", str(qb))
    b = bh // heads
    q, k, v = make_qkv(bh, sq, sk, d, seed=bh + sk, std=0.5 if d == 128 else 1.0, dtype=dtype)
    m = tail_mask(kind, b, sk, seed=sk + bh).to(TDT[dtype])
    kw = dict(mask=m.cuda(), causal=causal, want_lse=True)
    kv = None
    if extra == "philox":
        kw.update(drop_kind=capi.DROP_PHILOX, p_drop=0.1, seed=7, offset=3)
    elif extra == "kv_len":
        kv = torch.randint(0, sk + 1, (b,), generator=torch.Generator().manual_seed(5), dtype=torch.int32)
        kw.update(kv_len=kv.cuda())
    o, lse, _, _ = _run(q, k, v, **kw)
    o_all, lse_all, _, _ = _run(q, k, v, flags=capi.FLAG_NO_MASK_TRIM, **kw)
    assert torch.equal(o, o_all)
    assert torch.equal(lse, lse_all)
    if extra is None and bh <= 8:
        ref = oracle.attention(f32(q), f32(k), f32(v), mask=f32(m), causal=causal, want=("o", "lse"))
        assert np.abs(f32(o.cpu()) - ref["o"]).max() <= TOL[dtype]
        # one visible key: the LSE is that key's score, whose rounding (Q is rounded once after scaling)
        # goes with sum |q_i k_i| rather than with the score itself
        slack = 4.0 if kind == "last_live" else 1.0
        assert (np.abs(lse.cpu().numpy() - ref["lse"]) <= slack * LSE_TOL[dtype] + LSE_REL[dtype] * np.abs(ref["lse"])).all()


@pytest.mark.parametrize("bh,heads", [(8, 2), (512, 16)])
def test_skipped_key_tiles_are_never_read(bh, heads):
    """K and V rows in key tiles that hold only hard-masked keys may hold anything, NaN included: the
    forward does not visit them (unless told to, which is how this test knows that it tests something)."""
    s, d, b = 512, 64, bh // heads
    q, k, v = make_qkv(bh, s, s, d, seed=3)
    lens = torch.randint(1, s - 128, (b,), generator=torch.Generator().manual_seed(9))
    m = torch.zeros(b, 1, 1, s)
    k4, v4 = k.view(b, heads, s, d), v.view(b, heads, s, d)
    for i in range(b):
        m[i, ..., lens[i]:] = -10000.0
        first_unread = (int(lens[i]) + 127) // 128 * 128
        k4[i, :, first_unread:] = float("nan")
        v4[i, :, first_unread:] = float("nan")
    o = _run(q, k, v, mask=m.half().cuda())[0]
    assert not torch.isnan(o).any()
    o_all = _run(q, k, v, mask=m.half().cuda(), flags=capi.FLAG_NO_MASK_TRIM)[0]
    assert torch.isnan(o_all).view(b, -1).any(1).all()


def test_dropout_keeps_the_mean():
    """Kept probabilities are scaled by 256 / (256 - threshold), the reciprocal of the keep probability the
    8-bit threshold realises, so E[O] is the undropped O.  With q = 0 (uniform attention) and v = 1,
    O_i = scale * (kept keys of row i) / sk: the mean over 32 x 512 rows of 512 keys is 1 within 3 sigma
    of 8.4 million keep decisions -- the nominal factor 1 / (1 - p) would sit 15 sigma low at p = 0.1."""
    bh, s, d, p = 32, 512, 64, 0.1
    q = torch.zeros(bh, s, d, dtype=torch.float16, device="cuda")
    k = torch.randn(bh, s, d, device="cuda").half()
    v = torch.ones(bh, s, d, dtype=torch.float16, device="cuda")
    o, _, _, _ = _run(q, k, v, drop_kind=capi.DROP_PHILOX, p_drop=p, seed=77, offset=5)
    thr = capi.lib().fmha_drop_threshold(p)
    scale = capi.lib().fmha_drop_scale(p)
    assert thr == 26 and scale == pytest.approx(256 / 230, rel=1e-6)
    pk = (256 - thr) / 256
    sigma = scale * np.sqrt(pk * (1 - pk) / (bh * s * s))
    mean = o.float()[:, :, 0].double().mean().item()
    assert abs(mean - 1.0) <= 3 * sigma + 2e-5           # (+ the fp16 rounding of O near 1, averaged over the rows)
    assert abs(mean * (1 / (1 - p)) / scale - 1.0) > 6 * sigma   # what the nominal factor would have given


def test_drop_probability_below_one_step_is_no_dropout():
    """p < 1/512 rounds to a threshold of 0: nothing is dropped and nothing is scaled -- the call is the
    one without dropout, bit for bit, forward and backward."""
    q, k, v, do = (t.cuda() for t in make_qkv(4, 200, 300, 64, seed=8, with_dout=True))
    o0, l0, _, _ = _run(q, k, v, want_lse=True)
    o1, l1, _, _ = _run(q, k, v, want_lse=True, drop_kind=capi.DROP_PHILOX, p_drop=0.0015, seed=3)
    assert torch.equal(o0, o1) and torch.equal(l0, l1)
    g0 = capi.bwd(do, q, k, v, o0, l0)
    g1 = capi.bwd(do, q, k, v, o0, l0, drop_kind=capi.DROP_PHILOX, p_drop=0.0015, seed=3)
    assert all(torch.equal(a, b) for a, b in zip(g0, g1))
