"""The operators under HIP graph capture.

At the reference's shape a launch lasts 15-25 us, less than the host spends dispatching an operator,
so loops over such shapes are replayed from a captured graph.  The C ABI allocates nothing, never
synchronises and records no memset, which is what capture needs; this checks it: a captured train
step (forward with LSE and Philox dropout, backward) and the reference's three operators are
replayed several times on new input values, with eager work and synchronisations between the
replays, and every replay must reproduce the eager result bit for bit.
"""
import pytest
import torch

from conftest import make_qkv, pad_mask

pytestmark = pytest.mark.gpu


def _capture(fn):
    side = torch.cuda.Stream()          # default priority
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()                            # first calls outside capture: kernel attributes are set once per process
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        out = fn()
    return g, out


def test_train_step_replays_from_a_graph():
    from nvfuserexamples_amd import load_ops
    ops = load_ops()
    b, h, s, d = 4, 8, 320, 64
    q, k, v, do = (t.cuda() for t in make_qkv(b * h, s, s, d, seed=1, with_dout=True))
    m = pad_mask(b, s, s // 2, s).half().cuda()

    def step():
        o, lse = ops.fmha_fwd(q, k, v, m, 0.0, False, 0.1, 21, 6)
        return (o, lse) + tuple(ops.fmha_bwd(do, q, k, v, o, lse, m, 0.0, False, 0.1, 21, 6))

    g, outs = _capture(step)
    for r in range(4):
        fresh = [t.cuda() for t in make_qkv(b * h, s, s, d, seed=10 + r, with_dout=True)]
        for dst, src in zip((q, k, v, do), fresh):
            dst.copy_(src)
        g.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outs]
        want = step()                   # eager, same buffers
        torch.cuda.synchronize()
        for a, b_ in zip(got, want):
            assert torch.equal(a, b_), r


def test_reference_operators_replay_from_a_graph():
    import mha_manual  # noqa: F401
    ops = torch.ops.mha_manual
    bh, s, d = 64, 128, 64
    gen = torch.Generator(device="cuda").manual_seed(0)
    q, k, v = (torch.randn((bh, s, d), dtype=torch.half, device="cuda", generator=gen) for _ in range(3))
    amask = torch.empty((bh, s, s), device="cuda").random_(2, generator=gen).half()
    pad = torch.empty((bh, s, s), device="cuda").random_(2, generator=gen).half() * -1000
    dm = torch.empty((bh, s, s), device="cuda").random_(2, generator=gen).half()

    def calls():
        return [ops.fmha_nvfuser(q, k, v, amask), ops.fmha_train_nvfuser(q, k, v, pad, dm)] + \
            list(ops.fmha_train_saveim_nvfuser(q, k, v, pad, dm))

    g, outs = _capture(calls)
    for r in range(3):
        q.normal_(generator=gen)
        dm.random_(2, generator=gen)
        g.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outs]
        want = calls()
        torch.cuda.synchronize()
        for a, b_ in zip(got, want):
            assert torch.equal(a, b_), r


def test_decode_step_in_pieces_replays_from_a_graph():
    """A decode step whose key range runs in pieces (mask regrouping, the forward on the pieces, the merge; the
    operator allocates the workspace inside the capture) with valid key counts that change between replays."""
    from nvfuserexamples_amd import load_ops
    ops = load_ops()
    b, h, sk, d = 2, 4, 4096, 128
    q, k, v = (t.cuda() for t in make_qkv(b * h, 1, sk, d, seed=3, std=0.5))
    m = pad_mask(b, sk, sk // 2, sk).half().cuda()
    lens = torch.tensor([sk, sk // 3], dtype=torch.int32, device="cuda")

    def step():
        return ops.fmha_fwd(q, k, v, m, 0.0, False, 0.0, 0, 0, lens)

    g, outs = _capture(step)
    for r in range(4):
        fresh = [t.cuda() for t in make_qkv(b * h, 1, sk, d, seed=20 + r, std=0.5)]
        for dst, src in zip((q, k, v), fresh):
            dst.copy_(src)
        lens.copy_(torch.tensor([sk - 500 * r, 100 + 700 * r], dtype=torch.int32))
        g.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outs]
        want = step()
        torch.cuda.synchronize()
        for a, b_ in zip(got, want):
            assert torch.equal(a, b_), r


def test_noalloc_backward_replays_from_a_graph():
    """fmha_bwd_launch_noalloc is meant for callers under capture.  Its first call on a device looks up the
    address of the library's scratch array and sets kernel attributes, neither of which is a stream operation:
    that call happens eagerly (the warm-up inside _capture), then the launch is captured and replayed twice on
    new values, bit for bit equal to fmha_bwd_launch with a delta buffer of the caller's."""
    import ctypes as C
    from nvfuserexamples_amd import capi
    L = capi.lib()
    bh, s, d = 8, 320, 64
    q, k, v, do = (t.cuda() for t in make_qkv(bh, s, s, d, seed=2, with_dout=True))
    m = pad_mask(bh // 2, s, s // 2, s).half().cuda()
    o = torch.empty_like(q)
    lse = torch.empty(bh, s, dtype=torch.float32, device="cuda")
    got = [torch.empty_like(q) for _ in range(3)]
    ref = [torch.empty_like(q) for _ in range(3)]
    delta = torch.empty(bh, s, dtype=torch.float32, device="cuda")

    def params(grads, dl):
        P = capi.BwdParams()
        P.q, P.k, P.v, P.o, P.dout, P.lse = (t.data_ptr() for t in (q, k, v, o, do, lse))
        P.delta = dl.data_ptr() if dl is not None else None
        P.dq, P.dk, P.dv = (t.data_ptr() for t in grads)
        P.bh, P.sq, P.sk, P.d, P.dtype, P.scale = bh, s, s, d, capi.F16, d ** -0.5
        P.mask, P.mask_kind = m.data_ptr(), capi.MASK_ADDITIVE
        P.mask_bh_div, P.mask_stride_b, P.mask_stride_q = 2, s, 0
        P.drop_kind, P.p_drop, P.drop_scale, P.seed, P.offset = capi.DROP_PHILOX, 0.1, 0.0, 5, 7
        return P
    Pn, Pr = params(got, None), params(ref, delta)

    def forward():
        lse.copy_(capi.fwd(q, k, v, mask=m, want_lse=True, out=o, drop_kind=capi.DROP_PHILOX, p_drop=0.1, seed=5, offset=7)[1])

    def step():
        capi.check(L.fmha_bwd_launch_noalloc(C.byref(Pn), C.c_void_p(torch.cuda.current_stream().cuda_stream)))

    forward()
    g, _ = _capture(step)
    for r in range(2):
        for dst, src in zip((q, k, v, do), make_qkv(bh, s, s, d, seed=20 + r, with_dout=True)):
            dst.copy_(src.cuda())
        forward()
        for t in got:
            t.fill_(float("nan"))
        g.replay()
        capi.check(L.fmha_bwd_launch(C.byref(Pr), C.c_void_p(torch.cuda.current_stream().cuda_stream)))
        torch.cuda.synchronize()
        for a, b_ in zip(got, ref):
            assert torch.equal(a, b_), r
