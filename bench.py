#!/usr/bin/env python3
"""Headline benchmark: fused multi-head attention on one MI355X.

One "step" is one pass of the hot path over one batch of synthetic input, launched
through the C ABI (``libfmha_hip.so``) on torch's current HIP stream:

  workload "fwd"     BERT-large attention forward, B32 H16 S512 D64 fp16, additive
                     [B,1,1,S] padding mask (valid length U{256..512}), scale 1/8
  workload "fwdbwd"  the same shape as a train step: forward (saving the row
                     log-sum-exp) + backward, Philox dropout p=0.1

Inputs are resident in HBM before the timed region; several input sets are rotated
so that consecutive steps do not find their operands in the 256 MB last-level cache.
Prints ONE JSON line.  ``value`` is forward TFLOP/s (4*BH*S*S*D flops per step); the
train-step figure (14*BH*S*S*D) rides along under ``fwd_bwd``, and the long-sequence and
wide-head train-step configurations under ``configs``.

Timing protocol (every leg): W warm-up steps, then at least 0.3 s of the same steps so that the
board's clocks and power state settle (the kernels are power-limited: the first millisecond of a
cold run is not representative), then 25 blocks of exactly K steps each, every block bracketed by
HIP events on the launch stream and a device synchronisation; the MEDIAN block is reported
(``ms_per_step``), with the spread beside it.  ``roofline.launch_us`` is the same statistic over
blocks in which every launch has an event pair of its own (the figure comparable with rocprofv3's
per-kernel average); the step time exceeds it by the gap between back-to-back launches.

Work that is counted is work that is executed: the headline forward and train step run with
FMHA_FLAG_NO_MASK_TRIM, i.e. they visit every key tile of the dense shape the flop count is defined
on.  The library's default -- leaving out key tiles that the padding mask leaves without a live key,
with bit-identical results -- is timed beside them (``fwd_mask_trim``, ``fwd_bwd.mask_trim_*``).
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_MFMA_TFLOPS = 2500.0  # MI355X dense fp16/bf16 MFMA
PEAK_HBM_GBPS = 8000.0     # MI355X HBM3E
# HBM bytes per launch of the headline forward kernel (every key tile visited) as rocprofv3 counted them
# (FETCH_SIZE and WRITE_SIZE, each scaled by what the same counter reads for a 256 MiB copy in the same run):
# a counter reading of the build that was profiled, not something this script can measure.  It is read from
# a tracked file that names the commit it was taken at, so that a stale figure shows as such.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")
HEADLINE_KERNEL = "fmha_fwd_head_kernel<f16,QB2,per-key mask,no dropout>"


def measured_traffic(key):
    """(bytes per launch, commit the counters were read at) from profiles/traffic.json, or (None, None)."""
    try:
        with open(TRAFFIC_FILE) as f:
            e = json.load(f)[key]
        return int(e["bytes_per_launch"]), e.get("commit")
    except (OSError, KeyError, ValueError, TypeError):
        return None, None


B, H, S, D = 32, 16, 512, 64


def make_inputs(torch, capi, nsets, seed=0, train=False):
    g = torch.Generator().manual_seed(seed)
    sets = []
    for i in range(nsets):
        q, k, v = (torch.randn(B * H, S, D, generator=g).to(torch.float16).cuda() for _ in range(3))
        lens = torch.randint(S // 2, S + 1, (B,), generator=g)
        mask = torch.zeros(B, 1, 1, S)
        for b in range(B):
            mask[b, 0, 0, lens[b]:] = -10000.0
        mask = mask.to(torch.float16).cuda()
        d = dict(q=q, k=k, v=v, mask=mask, o=torch.empty_like(q))
        if train:
            d["dout"] = torch.randn(B * H, S, D, generator=g).to(torch.float16).cuda()
            d["lse"] = torch.empty(B * H, S, dtype=torch.float32, device="cuda")
            d["delta"] = torch.empty(B * H, S, dtype=torch.float32, device="cuda")
            d["dq"], d["dk"], d["dv"] = (torch.empty_like(q) for _ in range(3))
        sets.append(d)
    return sets


def fwd_params(capi, t, train=False, flags=0):
    P = capi.FwdParams()
    P.flags = flags
    P.q, P.k, P.v, P.o = (t[n].data_ptr() for n in ("q", "k", "v", "o"))
    P.mask, P.mask_kind = t["mask"].data_ptr(), capi.MASK_ADDITIVE
    P.mask_bh_div, P.mask_stride_b, P.mask_stride_q = H, S, 0
    P.bh, P.sq, P.sk, P.d = B * H, S, S, D
    P.dtype, P.scale = capi.F16, 0.125
    if train:
        P.lse = t["lse"].data_ptr()
        P.drop_kind, P.p_drop, P.drop_scale = capi.DROP_PHILOX, 0.1, 0.0  # 0: the mean-preserving factor
        P.seed, P.offset = 0x1234, 0
    return P


def bwd_params(capi, t, flags=0):
    P = capi.BwdParams()
    P.flags = flags
    for n in ("q", "k", "v", "o", "dout", "lse", "delta", "dq", "dk", "dv"):
        setattr(P, n, t[n].data_ptr())
    P.mask, P.mask_kind = t["mask"].data_ptr(), capi.MASK_ADDITIVE
    P.mask_bh_div, P.mask_stride_b, P.mask_stride_q = H, S, 0
    P.bh, P.sq, P.sk, P.d = B * H, S, S, D
    P.dtype, P.scale = capi.F16, 0.125
    P.drop_kind, P.p_drop, P.drop_scale = capi.DROP_PHILOX, 0.1, 0.0  # 0: the mean-preserving factor
    P.seed, P.offset = 0x1234, 0
    return P


BLOCKS = 25     # timed blocks per leg; the median block is reported
BURN_S = 0.3    # seconds of the same steps before timing, for clocks and power state to settle


def _median(xs):
    xs = sorted(xs)
    n = len(xs)
    return xs[n // 2] if n % 2 else 0.5 * (xs[n // 2 - 1] + xs[n // 2])


def settle(torch, step, warmup):
    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    t0, i = time.perf_counter(), warmup
    while time.perf_counter() - t0 < BURN_S:
        for _ in range(20):
            step(i)
            i += 1
        torch.cuda.synchronize()
    return i


def time_steps(torch, step, steps, warmup, blocks=BLOCKS, stats=None):
    """Median over `blocks` blocks of exactly `steps` steps each; HIP events on the stream the kernels are
    launched on (torch's current stream), a synchronisation either side of every block.  Returns
    (ms per step, host wall ms per step of the median block); `stats` receives the spread."""
    i0 = settle(torch, step, warmup)
    per, walls = [], []
    for b in range(blocks):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record()
        for i in range(steps):
            step(i0 + i)
        e1.record()
        torch.cuda.synchronize()
        walls.append((time.perf_counter() - t0) * 1e3 / steps)
        per.append(e0.elapsed_time(e1) / steps)
    if stats is not None:
        stats.update(blocks=blocks, steps_per_block=steps, block_ms_min=round(min(per), 5), block_ms_max=round(max(per), 5))
    return _median(per), _median(walls)


def time_launches(torch, step, steps, warmup, blocks=BLOCKS):
    """Duration of ONE launch: a HIP event pair around every launch (same stream as the kernels), averaged
    over a block of `steps` launches; the median block.  Excludes the idle gap between back-to-back
    launches, so it is the figure comparable with rocprofv3's per-kernel average."""
    i0 = settle(torch, step, warmup)
    per = []
    for b in range(blocks):
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        for i, (a, c) in enumerate(ev):
            a.record()
            step(i0 + i)
            c.record()
        torch.cuda.synchronize()
        per.append(sum(a.elapsed_time(c) for a, c in ev) / steps)
    return _median(per)


def short_sequence_legs(torch, capi, L, stream, steps, warmup):
    """The bandwidth-bound shapes: the reference's own operators at the reference's fixed shape
    (BH 512, S 128, D 64 with full [BH,S,S] mask tensors: fmha/fmha_manual.cpp:24-29, test.py:20-23),
    the same operators with their full mask tensors at the headline sequence length (S 512), a train
    step at the short shape, and the BERT-base configuration that the CPU baseline is timed on.
    Reported as time and as algorithmic bytes per second against the HBM peak, beside the headline,
    never as `value`.  The legs rotate input sets that together exceed the 256 MB last-level cache;
    the BERT-base leg is 6 MB and stays cache-resident whatever is rotated."""
    legs = {}

    def run(name, Ps, nbytes, note):
        def step(i):
            L.fmha_fwd_launch(C.byref(Ps[i % len(Ps)]), stream)
        capi.check(L.fmha_fwd_launch(C.byref(Ps[0]), stream))
        ms, _ = time_steps(torch, step, steps, warmup)
        legs[name] = {"us": round(ms * 1e3, 2), "algorithmic_MB": round(nbytes / 1e6, 2),
                      "hbm_GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
                      "hbm_frac": round(nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4), "inputs": note}

    g = torch.Generator().manual_seed(7)
    bh, s, d = 512, 128, 64
    keep, infer, train, save = [], [], [], []
    for _ in range(6):
        q, k, v = (torch.randn(bh, s, d, generator=g).to(torch.float16).cuda() for _ in range(3))
        o = torch.empty_like(q)
        amask = (torch.rand(bh, s, s, generator=g) > 0.1).to(torch.float16).cuda()
        pad = (torch.rand(bh, s, s, generator=g) > 0.9).to(torch.float16).mul_(-1000.0).cuda()
        dm = (torch.rand(bh, s, s, generator=g) > 0.5).to(torch.float16).cuda()
        sm, dr = (torch.empty(bh, s, s, dtype=torch.float16, device="cuda") for _ in range(2))
        keep.append((q, k, v, o, amask, pad, dm, sm, dr))
        for kind in ("infer", "train", "save"):
            P = capi.FwdParams()
            P.q, P.k, P.v, P.o = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr()
            P.bh, P.sq, P.sk, P.d = bh, s, s, d
            P.dtype, P.scale = capi.F16, 0.125
            P.mask_bh_div, P.mask_stride_b, P.mask_stride_q = 1, s * s, s
            if kind == "infer":
                P.mask, P.mask_kind, P.mask_neg = amask.data_ptr(), capi.MASK_KEEP01, -10000.0
                infer.append(P)
            else:
                P.mask, P.mask_kind = pad.data_ptr(), capi.MASK_ADDITIVE
                P.drop_kind, P.drop_mask, P.drop_scale = capi.DROP_TENSOR, dm.data_ptr(), 2.0
                if kind == "save":
                    P.save_softmax, P.save_dropout = sm.data_ptr(), dr.data_ptr()
                (save if kind == "save" else train).append(P)
    run("fmha_nvfuser_BH512_S128_D64_full_mask", infer, 4 * bh * s * d * 2 + bh * s * s * 2, "6 sets rotated")
    run("fmha_train_nvfuser_BH512_S128_D64_full_masks", train, 4 * bh * s * d * 2 + 2 * bh * s * s * 2,
        "6 sets rotated")
    run("fmha_train_saveim_nvfuser_BH512_S128_D64_full_masks", save, 4 * bh * s * d * 2 + 4 * bh * s * s * 2,
        "6 sets rotated")
    del keep, infer, train, save

    # the same two operators at the headline sequence length (S 512): 403 / 671 MB per call, two sets rotated
    s5 = 512
    keep5, infer5, train5, save5 = [], [], [], []
    for _ in range(2):
        q, k, v = (torch.randn(bh, s5, d, generator=g).to(torch.float16).cuda() for _ in range(3))
        o = torch.empty_like(q)
        amask = (torch.rand(bh, s5, s5, generator=g) > 0.1).to(torch.float16).cuda()
        pad = (torch.rand(bh, s5, s5, generator=g) > 0.9).to(torch.float16).mul_(-1000.0).cuda()
        dm = (torch.rand(bh, s5, s5, generator=g) > 0.5).to(torch.float16).cuda()
        sm, dr = (torch.empty(bh, s5, s5, dtype=torch.float16, device="cuda") for _ in range(2))
        lse5 = torch.empty(bh, s5, dtype=torch.float32, device="cuda")
        keep5.append((q, k, v, o, amask, pad, dm, sm, dr, lse5))
        for kind in ("infer", "train", "save"):
            P = capi.FwdParams()
            P.q, P.k, P.v, P.o = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr()
            P.bh, P.sq, P.sk, P.d = bh, s5, s5, d
            P.dtype, P.scale = capi.F16, 0.125
            P.mask_bh_div, P.mask_stride_b, P.mask_stride_q = 1, s5 * s5, s5
            if kind == "infer":
                P.mask, P.mask_kind, P.mask_neg = amask.data_ptr(), capi.MASK_KEEP01, -10000.0
                infer5.append(P)
            else:
                P.mask, P.mask_kind = pad.data_ptr(), capi.MASK_ADDITIVE
                P.drop_kind, P.drop_mask, P.drop_scale = capi.DROP_TENSOR, dm.data_ptr(), 2.0
                if kind == "save":  # (with an LSE buffer: the forward, then one streaming launch for both saved tensors)
                    P.save_softmax, P.save_dropout, P.lse = sm.data_ptr(), dr.data_ptr(), lse5.data_ptr()
                (save5 if kind == "save" else train5).append(P)
    run("fmha_nvfuser_BH512_S512_D64_full_mask", infer5, 4 * bh * s5 * d * 2 + bh * s5 * s5 * 2, "2 sets rotated")
    run("fmha_train_nvfuser_BH512_S512_D64_full_masks", train5, 4 * bh * s5 * d * 2 + 2 * bh * s5 * s5 * 2,
        "2 sets rotated")
    run("fmha_train_saveim_nvfuser_BH512_S512_D64_full_masks", save5, 4 * bh * s5 * d * 2 + 4 * bh * s5 * s5 * 2,
        "2 sets rotated")
    del keep5, infer5, train5, save5

    # train step at the same short shape (the reference has no backward): [B,1,1,S] padding mask, Philox
    # dropout; forward with LSE, then the one-launch short-sequence backward
    bb = 32
    tkeep, tsteps = [], []
    for _ in range(6):
        t = {n: torch.randn(bh, s, d, generator=g).to(torch.float16).cuda() for n in ("q", "k", "v", "dout")}
        for n in ("o", "dq", "dk", "dv"):
            t[n] = torch.empty_like(t["q"])
        t["lse"], t["delta"] = (torch.empty(bh, s, dtype=torch.float32, device="cuda") for _ in range(2))
        m = torch.zeros(bb, 1, 1, s)
        for i in range(bb):
            m[i, 0, 0, 64 + 2 * i:] = -10000.0
        t["mask"] = m.to(torch.float16).cuda()
        F, Bp = capi.FwdParams(), capi.BwdParams()
        for P in (F, Bp):
            P.q, P.k, P.v, P.o, P.lse = (t[n].data_ptr() for n in ("q", "k", "v", "o", "lse"))
            P.bh, P.sq, P.sk, P.d = bh, s, s, d
            P.dtype, P.scale = capi.F16, 0.125
            P.mask, P.mask_kind = t["mask"].data_ptr(), capi.MASK_ADDITIVE
            P.mask_bh_div, P.mask_stride_b, P.mask_stride_q = bh // bb, s, 0
            P.drop_kind, P.p_drop, P.drop_scale, P.seed, P.offset = capi.DROP_PHILOX, 0.1, 0.0, 0x1234, 0
        Bp.dout, Bp.delta, Bp.dq, Bp.dk, Bp.dv = (t[n].data_ptr() for n in ("dout", "delta", "dq", "dk", "dv"))
        tkeep.append(t)
        tsteps.append((F, Bp))

    def train_step(i):
        F, Bp = tsteps[i % len(tsteps)]
        L.fmha_fwd_launch(C.byref(F), stream)
        L.fmha_bwd_launch(C.byref(Bp), stream)
    capi.check(L.fmha_fwd_launch(C.byref(tsteps[0][0]), stream))
    capi.check(L.fmha_bwd_launch(C.byref(tsteps[0][1]), stream))
    ms, _ = time_steps(torch, train_step, steps, warmup)
    nbytes = 12 * bh * s * d * 2 + 3 * bh * s * 4 + bb * s * 2 * 2
    legs["train_step_BH512_S128_D64_pad_mask_dropout"] = {
        "us": round(ms * 1e3, 2), "algorithmic_MB": round(nbytes / 1e6, 2),
        "hbm_GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
        "hbm_frac": round(nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4),
        "tflops": round(14.0 * bh * s * s * d / (ms * 1e-3) / 1e12, 2), "inputs": "6 sets rotated"}
    del tkeep, tsteps

    b1, h1 = 8, 12   # BERT-base forward: the configuration of the CPU baseline
    q1, k1, v1 = (torch.randn(b1 * h1, s, d, generator=g).to(torch.float16).cuda() for _ in range(3))
    o1 = torch.empty_like(q1)
    m1 = torch.zeros(b1, 1, 1, s)
    for i in range(b1):
        m1[i, 0, 0, 64 + 8 * i:] = -10000.0
    m1 = m1.to(torch.float16).cuda()
    P = capi.FwdParams()
    P.q, P.k, P.v, P.o = q1.data_ptr(), k1.data_ptr(), v1.data_ptr(), o1.data_ptr()
    P.bh, P.sq, P.sk, P.d = b1 * h1, s, s, d
    P.dtype, P.scale = capi.F16, 0.125
    P.mask, P.mask_kind = m1.data_ptr(), capi.MASK_ADDITIVE
    P.mask_bh_div, P.mask_stride_b, P.mask_stride_q = h1, s, 0
    name = "B8_H12_S128_D64_pad_mask"
    run(name, [P], 4 * b1 * h1 * s * d * 2 + b1 * s * 2, "one set, cache-resident")
    legs[name]["tflops"] = round(4.0 * b1 * h1 * s * s * d / (legs[name]["us"] * 1e-6) / 1e12, 2)
    return legs


def operator_legs(torch, steps, warmup):
    """The reference's three operators as a caller sees them (torch.ops.mha_manual.*, outputs
    allocated per call) at the reference's shape, timed per call on the host clock: called eagerly
    back to back, and replayed from a captured HIP graph.  One input set (the point is the host's
    share, not HBM): a launch lasts 15-25 us here, about what dispatching an operator costs."""
    from nvfuserexamples_amd import load_ops
    ops = load_ops()
    bh, s, d = 512, 128, 64
    g = torch.Generator(device="cuda").manual_seed(3)
    q, k, v = (torch.randn((bh, s, d), dtype=torch.float16, device="cuda", generator=g) for _ in range(3))
    amask = torch.empty((bh, s, s), device="cuda").random_(2, generator=g).half()
    pad = torch.empty((bh, s, s), device="cuda").random_(2, generator=g).half() * -1000
    dm = torch.empty((bh, s, s), device="cuda").random_(2, generator=g).half()
    calls = {"fmha_nvfuser": lambda: ops.fmha_nvfuser(q, k, v, amask),
             "fmha_train_nvfuser": lambda: ops.fmha_train_nvfuser(q, k, v, pad, dm),
             "fmha_train_saveim_nvfuser": lambda: ops.fmha_train_saveim_nvfuser(q, k, v, pad, dm)}
    legs = {}
    for name, fn in calls.items():
        _, eager_ms = time_steps(torch, lambda i: fn(), steps, warmup)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            keep = fn()
        _, graph_ms = time_steps(torch, lambda i: graph.replay(), steps, warmup)
        legs[name] = {"eager_us_per_call": round(eager_ms * 1e3, 2), "graph_replay_us_per_call": round(graph_ms * 1e3, 2)}
        del graph, keep
    # the reference's own protocol on the same operators and inputs (reference perf_measurement.py:29-50,
    # perf_measurement_train.py:35-60): 10 warm-up calls, then 1000 calls under no_grad between two events
    # on the current stream, one input set, outputs allocated per call
    for name, fn in calls.items():
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        with torch.no_grad():
            for _ in range(10):
                fn()
            start.record()
            for _ in range(1000):
                fn()
            stop.record()
        start.synchronize()
        stop.synchronize()
        legs[name]["reference_protocol_us_per_call"] = round(start.elapsed_time(stop), 2)  # ms / 1000 calls = us per call
    legs["reference_protocol"] = "10 warm-up + 1000 timed calls of torch.ops.mha_manual.<op> under no_grad between two events"
    return legs


def head_dim_256_leg(torch, capi):
    """Head dim 256 (built for coverage, not tuned): forward and backward at BH 128, S 2048, fp16, no mask."""
    bh, s, d = 128, 2048, 256
    g = torch.Generator().manual_seed(3)
    q, k, v, do = ((torch.randn(bh, s, d, generator=g) * 0.35).to(torch.float16).cuda() for _ in range(4))
    o, lse, _, _ = capi.fwd(q, k, v, want_lse=True)
    grads = capi.bwd(do, q, k, v, o, lse)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
    torch.cuda.synchronize()
    n = 5
    ev[0].record()
    for _ in range(n):
        capi.fwd(q, k, v, want_lse=True, out=o)
    ev[1].record()
    for _ in range(n):
        capi.bwd(do, q, k, v, o, lse, grads=grads)
    ev[2].record()
    torch.cuda.synchronize()
    f_ms, b_ms = ev[0].elapsed_time(ev[1]) / n, ev[1].elapsed_time(ev[2]) / n
    flops = 4.0 * bh * s * s * d
    return {"workload": "BH128 S2048 D256 fp16, no mask (includes the wrappers' output allocation where they allocate)",
            "fwd_us": round(f_ms * 1e3, 1), "fwd_tflops": round(flops / (f_ms * 1e-3) / 1e12, 1),
            "bwd_us": round(b_ms * 1e3, 1), "bwd_tflops": round(2.5 * flops / (b_ms * 1e-3) / 1e12, 1)}


def config_leg(torch, capi, L, stream, steps, warmup, b, h, s, d, dtype, causal, p_drop, std, nsets):
    """Forward, backward and train step of one benchmark configuration (no padding mask), through the C ABI.
    Flops: 4 / 10 / 14 * BH*S*S*D, times (S+1)/(2S) under the causal mask (the tiles above the diagonal are
    neither counted nor visited).  Bytes: forward 4*BH*S*D*e + BH*S*4 (LSE), backward 8*BH*S*D*e + 2*BH*S*4."""
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    bh = b * h
    g = torch.Generator().manual_seed(11)
    sets = []
    for _ in range(nsets):
        t = {n: (torch.randn(bh, s, d, generator=g) * std).to(tdt).cuda() for n in ("q", "k", "v", "dout")}
        for n in ("o", "dq", "dk", "dv"):
            t[n] = torch.empty_like(t["q"])
        t["lse"], t["delta"] = (torch.empty(bh, s, dtype=torch.float32, device="cuda") for _ in range(2))
        F, Bp = capi.FwdParams(), capi.BwdParams()
        for P in (F, Bp):
            P.q, P.k, P.v, P.o, P.lse = (t[n].data_ptr() for n in ("q", "k", "v", "o", "lse"))
            P.bh, P.sq, P.sk, P.d = bh, s, s, d
            P.dtype, P.scale, P.causal = (capi.F16 if dtype == "f16" else capi.BF16), d ** -0.5, int(causal)
            if p_drop:
                P.drop_kind, P.p_drop, P.drop_scale, P.seed, P.offset = capi.DROP_PHILOX, p_drop, 0.0, 0x1234, 0
        Bp.dout, Bp.delta, Bp.dq, Bp.dk, Bp.dv = (t[n].data_ptr() for n in ("dout", "delta", "dq", "dk", "dv"))
        sets.append((t, F, Bp))
    capi.check(L.fmha_fwd_launch(C.byref(sets[0][1]), stream))
    capi.check(L.fmha_bwd_launch(C.byref(sets[0][2]), stream))

    def fwd(i):
        if L.fmha_fwd_launch(C.byref(sets[i % nsets][1]), stream):
            raise RuntimeError("forward launch refused inside a timed region")

    def bwd(i):
        if L.fmha_bwd_launch(C.byref(sets[i % nsets][2]), stream):
            raise RuntimeError("backward launch refused inside a timed region")

    def both(i):
        fwd(i)
        bwd(i)
    for _, F, _ in sets:   # every set's O and LSE must exist before its backward is timed alone
        L.fmha_fwd_launch(C.byref(F), stream)
    n = max(5, steps // 4) if s * s * bh > 2 ** 27 else steps
    blocks = 9 if s * s * bh * d > 2 ** 34 else BLOCKS
    ms_f, _ = time_steps(torch, fwd, n, warmup, blocks)
    ms_b, _ = time_steps(torch, bwd, n, warmup, blocks)
    ms_t, _ = time_steps(torch, both, n, warmup, blocks)
    dense = float(bh) * s * s * d
    cf = (s + 1) / (2.0 * s) if causal else 1.0
    e = 2
    by_f = 4.0 * bh * s * d * e + bh * s * 4
    by_b = 8.0 * bh * s * d * e + 2 * bh * s * 4

    def part(ms, fl, by):
        tf = fl * cf / (ms * 1e-3) / 1e12
        return {"us": round(ms * 1e3, 1), "tflops": round(tf, 1), "mfma_frac": round(tf / PEAK_MFMA_TFLOPS, 4),
                "hbm_GBps": round(by / (ms * 1e-3) / 1e9, 1), "hbm_frac": round(by / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4)}
    out = {"workload": f"B{b} H{h} S{s} D{d} {dtype}, {'causal mask' if causal else 'no mask'}, "
                       f"{'Philox dropout p=%g' % p_drop if p_drop else 'no dropout'}; {nsets} input set(s) rotated",
           "flops_counted": "causal count: dense x (S+1)/(2S)" if causal else "dense",
           "fwd": part(ms_f, 4 * dense, by_f), "bwd": part(ms_b, 10 * dense, by_b),
           "fwd_bwd": part(ms_t, 14 * dense, by_f + by_b), "steps_per_block": n, "blocks": blocks}
    if causal:
        out["fwd_bwd"]["tflops_full_count"] = round(14 * dense / (ms_t * 1e-3) / 1e12, 1)
    return out


def fp8_leg(torch, capi, L, stream, steps, warmup):
    """The e4m3 forward (a separate operator) at the headline shape with the same padding masks: time and
    TFLOP/s against the dense fp8 MFMA peak.  Never part of `value`."""
    g = torch.Generator().manual_seed(21)
    sets = []
    for _ in range(4):
        q8, k8, v8 = (torch.randn(B * H, S, D, generator=g).to(torch.float8_e4m3fn).cuda() for _ in range(3))
        lens = torch.randint(S // 2, S + 1, (B,), generator=g)
        mask = torch.zeros(B, 1, 1, S)
        for b in range(B):
            mask[b, 0, 0, lens[b]:] = -10000.0
        mask = mask.half().cuda()
        o = torch.empty(B * H, S, D, dtype=torch.float16, device="cuda")
        P = capi.FwdFp8Params()
        P.q, P.k, P.v, P.o = q8.data_ptr(), k8.data_ptr(), v8.data_ptr(), o.data_ptr()
        P.mask, P.mask_bh_div, P.mask_stride_b = mask.data_ptr(), H, S
        P.bh, P.sq, P.sk, P.d = B * H, S, S, D
        P.out_dtype, P.scale = capi.F16, 0.125
        P.descale_q = P.descale_k = P.descale_v = 1.0
        sets.append((P, q8, k8, v8, mask, o))
    capi.check(L.fmha_fwd_fp8_launch(C.byref(sets[0][0]), stream))

    def step(i):
        L.fmha_fwd_fp8_launch(C.byref(sets[i % len(sets)][0]), stream)
    ms, _ = time_steps(torch, step, steps, warmup)
    fl = 4.0 * B * H * S * S * D
    by = 3.0 * B * H * S * D + B * H * S * D * 2 + B * S * 2
    return {"workload": "B32 H16 S512 D64, q/k/v e4m3, O fp16, [B,1,1,S] padding mask; 4 input sets rotated",
            "us": round(ms * 1e3, 2), "tflops": round(fl / (ms * 1e-3) / 1e12, 1),
            "frac_of_fp8_mfma_peak": round(fl / (ms * 1e-3) / 1e12 / 5000.0, 4),
            "hbm_frac": round(by / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4)}


DECODE_SHAPES = {  # name: (heads, query rows, keys, head dim)
    "BH32_Sk32768_D128": (32, 1, 32768, 128),
    "BH64_Sk8192_D128": (64, 1, 8192, 128),
    "BH8_Sk131072_D128": (8, 1, 131072, 128),
    "BH128_Sk16384_D64": (128, 1, 16384, 64),
    "BH512_Sk4096_D128": (512, 1, 4096, 128),   # enough heads to fill the chip: never cut
}


def decode_sets(torch, bh, sq, sk, d):
    """Input sets for a decode step, enough of them that K and V (the bytes that count) come from HBM."""
    g = torch.Generator().manual_seed(31)
    nset = max(2, int(600e6 // (4 * bh * sk * d)) + 1)
    sets = []
    for _ in range(nset):
        q = torch.randn(bh, sq, d, generator=g).half().cuda()
        k, v = (torch.randn(bh, sk, d, device="cuda", dtype=torch.float16) for _ in range(2))
        sets.append((q, k, v, torch.empty_like(q)))
    return sets


def decode_leg(torch, capi, steps, warmup):
    """Decode steps (one query row per head against a long fp16 K/V cache, no mask) on the decode kernel: HBM-bound,
    the bytes are K and V once.  `plain` is the launch by head, `pieces` the same call with a workspace, where the
    library cuts the key range so that the whole chip streams (not needed, and not done, with enough heads).
    Never part of `value`."""
    out = {}
    for name, (bh, sq, sk, d) in DECODE_SHAPES.items():
        sets = decode_sets(torch, bh, sq, sk, d)
        ws = torch.empty(64 << 20, dtype=torch.uint8, device="cuda")
        by = 4.0 * bh * sk * d + 4.0 * bh * sq * d
        leg = {"workload": f"bh {bh}, {sq} query row, {sk} keys, head dim {d}, fp16; {len(sets)} input sets rotated",
               "algorithmic_MB": round(by / 1e6, 1)}
        for mode, w in (("plain", False), ("pieces", ws)):
            def step(i):
                q, k, v, o = sets[i % len(sets)]
                capi.fwd(q, k, v, out=o, workspace=w)
            ms, _ = time_steps(torch, step, steps, warmup, blocks=9)
            leg[mode] = {"us": round(ms * 1e3, 1), "TBps": round(by / (ms * 1e-3) / 1e12, 2),
                         "hbm_frac": round(by / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 3)}
        out[name] = leg
        del sets, ws
    # the same steps on an e4m3 cache (q, k, v e4m3, O fp16): half the bytes
    for name in ("BH32_Sk32768_D128", "BH512_Sk4096_D128"):
        bh, sq, sk, d = DECODE_SHAPES[name]
        nset = max(2, int(600e6 // (2 * bh * sk * d)) + 1)
        sets = [tuple(torch.randn(bh, s_, d, device="cuda").to(torch.float8_e4m3fn) for s_ in (sq, sk, sk))
                for _ in range(nset)]
        ws = torch.empty(64 << 20, dtype=torch.uint8, device="cuda")
        by = 2.0 * bh * sk * d + bh * sq * d * 3.0

        def step8(i):
            q8, k8, v8 = sets[i % len(sets)]
            capi.fwd_fp8(q8, k8, v8, workspace=ws)
        ms, _ = time_steps(torch, step8, steps, warmup, blocks=9)
        out[name]["e4m3_cache"] = {"us": round(ms * 1e3, 1), "algorithmic_MB": round(by / 1e6, 1),
                                   "TBps": round(by / (ms * 1e-3) / 1e12, 2),
                                   "hbm_frac": round(by / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 3)}
        del sets, ws
    return out


def profile_leg(torch, capi, L, stream, args):
    """`--profile LEG`: nothing but LEG's launches, `--steps` times after `--warmup`, for a run under
    `rocprofv3` (kernel trace or counters) in which every dispatch of a kernel belongs to one workload.
    Prints a one-line note instead of the benchmark line."""
    leg = args.profile
    steps = []
    keep = []
    if leg in ("fwd", "fwd_trim", "train"):
        train = leg.startswith("train")
        sets = make_inputs(torch, capi, args.sets, seed=1 if train else 0, train=train)
        flags = 0 if leg == "fwd_trim" else capi.FLAG_NO_MASK_TRIM
        F = [fwd_params(capi, t, train=train, flags=flags) for t in sets]
        steps.append(lambda i: L.fmha_fwd_launch(C.byref(F[i % len(F)]), stream))
        keep += [sets, F]
        if train:
            Bp = [bwd_params(capi, t, flags=flags) for t in sets]
            steps.append(lambda i: L.fmha_bwd_launch(C.byref(Bp[i % len(Bp)]), stream))
            keep.append(Bp)
    elif leg in ("c4", "c5", "d256"):
        b, h, s, d, dt, causal, p, std = {"c4": (4, 16, 2048, 64, torch.float16, False, 0.1, 1.0),
                                          "c5": (16, 32, 1024, 128, torch.bfloat16, True, 0.0, 0.5),
                                          "d256": (8, 16, 2048, 256, torch.float16, False, 0.0, 0.35)}[leg]
        g = torch.Generator().manual_seed(11)
        q, k, v, do = ((torch.randn(b * h, s, d, generator=g) * std).to(dt).cuda() for _ in range(4))
        kw = dict(causal=causal)
        if p:
            kw.update(drop_kind=capi.DROP_PHILOX, p_drop=p, seed=0x1234, offset=0)
        o, lse = capi.fwd(q, k, v, want_lse=True, **kw)[:2]
        grads = tuple(torch.empty_like(q) for _ in range(3))
        delta = torch.empty_like(lse)
        steps.append(lambda i: capi.fwd(q, k, v, want_lse=True, out=o, **kw))
        steps.append(lambda i: capi.bwd(do, q, k, v, o, lse, grads=grads, delta=delta, **kw))
    elif leg in ("decode", "decode_plain"):
        sets = decode_sets(torch, *DECODE_SHAPES["BH32_Sk32768_D128"])
        ws = torch.empty(64 << 20, dtype=torch.uint8, device="cuda") if leg == "decode" else False

        def decode_step(i):
            q, k, v, o = sets[i % len(sets)]
            capi.fwd(q, k, v, out=o, workspace=ws)
        steps.append(decode_step)
    elif leg == "fp8":
        g = torch.Generator().manual_seed(21)
        q8, k8, v8 = (torch.randn(B * H, S, D, generator=g).to(torch.float8_e4m3fn).cuda() for _ in range(3))
        mask = torch.zeros(B, 1, 1, S)
        for b_, n_ in enumerate(torch.randint(S // 2, S + 1, (B,), generator=g).tolist()):
            mask[b_, 0, 0, n_:] = -10000.0
        mask = mask.half().cuda()
        steps.append(lambda i: capi.fwd_fp8(q8, k8, v8, mask=mask, scale=0.125))
    else:
        print(f"bench.py: unknown --profile leg {leg!r}", file=sys.stderr)
        return 2
    for i in range(args.warmup + args.steps):
        for st in steps:
            st(i)
    torch.cuda.synchronize()
    print(json.dumps({"profile_leg": leg, "steps": args.steps, "warmup": args.warmup}))
    return 0


def torch_sdpa_context(torch, steps, warmup):
    """For scale only: PyTorch's own fused attention (torch.nn.functional.scaled_dot_product_attention,
    whichever backend it selects) on the same GPU at the headline shape, [B,H,S,D] fp16 tensors -- the
    same padding mask for the forward, and a forward + backward with dropout 0.1 (no mask, which its
    fastest backend requires).  Not a baseline of the reference and not part of `value`."""
    import torch.nn.functional as F
    out = {}
    try:
        g = torch.Generator(device="cuda").manual_seed(5)
        q, k, v = (torch.randn((B, H, S, D), dtype=torch.float16, device="cuda", generator=g) for _ in range(3))
        m = torch.zeros(B, 1, 1, S, dtype=torch.float16, device="cuda")
        for i in range(B):
            m[i, 0, 0, 256 + 8 * i:] = -10000.0
        with torch.no_grad():
            ms, _ = time_steps(torch, lambda i: F.scaled_dot_product_attention(q, k, v, attn_mask=m), steps, warmup)
            ms_nomask, _ = time_steps(torch, lambda i: F.scaled_dot_product_attention(q, k, v), steps, warmup)
        out["fwd_pad_mask_us"] = round(ms * 1e3, 1)
        out["fwd_no_mask_us"] = round(ms_nomask * 1e3, 1)
        out["fwd_no_mask_tflops"] = round(4.0 * B * H * S * S * D / (ms_nomask * 1e-3) / 1e12, 1)
        qg, kg, vg = (t.clone().requires_grad_(True) for t in (q, k, v))
        do = torch.randn_like(q)

        def step(i):
            o = F.scaled_dot_product_attention(qg, kg, vg, dropout_p=0.1)
            o.backward(do)
        n = max(10, steps // 10)
        ms_t, _ = time_steps(torch, step, n, max(2, warmup // 10))
        out["train_step_dropout_us"] = round(ms_t * 1e3, 1)
        out["train_step_tflops"] = round(14.0 * B * H * S * S * D / (ms_t * 1e-3) / 1e12, 1)
        out["torch"] = torch.__version__
        # a decode step (the first shape of `decode_steps`: 2 x 16 heads, one query row, 32 768 keys, D 128)
        del qg, kg, vg, do
        qd = torch.randn((2, 16, 1, 128), dtype=torch.float16, device="cuda", generator=g)
        kvs = [tuple(torch.randn((2, 16, 32768, 128), dtype=torch.float16, device="cuda", generator=g) for _ in range(2))
               for _ in range(3)]
        with torch.no_grad():
            ms_d, _ = time_steps(torch, lambda i: F.scaled_dot_product_attention(qd, *kvs[i % 3]), max(10, steps // 2),
                                 max(2, warmup // 2), blocks=9)
        out["decode_BH32_Sk32768_D128_us"] = round(ms_d * 1e3, 1)
    except Exception as e:  # a context figure must never break the benchmark
        out["unavailable"] = repr(e)[:200]
    return out


def smi_sample():
    """One reading of socket power and graphics clocks from the board's management firmware (amd-smi), or None."""
    import re
    import shutil
    import subprocess
    exe = shutil.which("amd-smi") or "/opt/rocm/bin/amd-smi"
    if not os.path.exists(exe):
        return None
    try:
        r = subprocess.run([exe, "metric", "-g", "0", "-c", "-p"], stdout=subprocess.PIPE,
                           stderr=subprocess.DEVNULL, text=True, timeout=20)
    except Exception:
        return None
    pw = re.search(r"SOCKET_POWER:\s*(\d+)\s*W", r.stdout)
    clk = [int(m) for m in re.findall(r"GFX_\d+:\s*\n\s*CLK:\s*(\d+)\s*MHz", r.stdout)]
    mx = re.search(r"MAX_CLK:\s*(\d+)\s*MHz", r.stdout)
    if not pw or not clk:
        return None
    return {"socket_power_w": int(pw.group(1)), "gfx_clk_mhz_mean": round(sum(clk) / len(clk)),
            "gfx_clk_mhz_min": min(clk), "gfx_max_clk_mhz": int(mx.group(1)) if mx else None}


def power_probe(torch, step, idle, seconds=2.0):
    """Socket power and graphics clocks as the board's management firmware reports them (amd-smi),
    sampled while `step` runs back to back on a second thread; `idle` is a reading taken before the
    process touched the GPU.  The firmware's clock is the frequency it has set (a target, read at one
    instant per die); the clock the waves really saw is `effective_core_clock_mhz` (cycle counter over the
    100 MHz counter inside the kernel).  Returns None where the tool is missing or its output has no such fields."""
    import threading
    sample = smi_sample
    torch.cuda.synchronize()
    stop = [False]

    def load():
        i = 0
        while not stop[0]:
            for _ in range(100):
                step(i)
                i += 1
            torch.cuda.synchronize()

    th = threading.Thread(target=load)
    th.start()
    busy = []
    t_end = time.perf_counter() + seconds
    time.sleep(0.5)
    while time.perf_counter() < t_end:
        b = sample()
        if b:
            busy.append(b)
    stop[0] = True
    th.join()
    if not idle or not busy:
        return None
    top = max(busy, key=lambda b: b["socket_power_w"])
    return {"tool": "amd-smi metric -c -p: idle before the process's first GPU work, busy while the headline kernel runs back to back",
            "idle_socket_power_w": idle["socket_power_w"], "busy_socket_power_w": top["socket_power_w"],
            "busy_gfx_clk_mhz_mean": top["gfx_clk_mhz_mean"], "busy_gfx_clk_mhz_min": top["gfx_clk_mhz_min"],
            "gfx_max_clk_mhz": top["gfx_max_clk_mhz"], "samples": len(busy)}


def _cpu_eager_leg(torch, b, h, s, d, lo, budget_s, min_iters):
    """The reference's eager composition (its ground truth, reference test.py:12-18: matmul, mask add, softmax,
    matmul) on the host cores in fp32: b sequences of h heads, padding mask with valid lengths U{lo..s}; 3 warm-up
    calls, then calls until both `min_iters` and `budget_s` seconds are reached."""
    from oracle import eager
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(b * h, s, d, generator=g) for _ in range(3))
    lens = torch.randint(lo, s + 1, (b,), generator=g)
    keep = torch.zeros(b, 1, s)
    for i in range(b):
        keep[i, 0, :lens[i]] = 1.0
    keep = keep.repeat_interleave(h, 0)  # [bh,1,s] 0/1 mask as the inference op takes it
    for _ in range(3):
        eager.infer_mha(q, k, v, keep)
    n, t0 = 0, time.perf_counter()
    while True:
        eager.infer_mha(q, k, v, keep)
        n += 1
        el = time.perf_counter() - t0
        if (el > budget_s and n >= min_iters) or n >= 2000000:
            break
    return n, el, 4.0 * b * h * s * s * d


def pipe_ceilings(torch, capi, L, stream, fwd_params_of, time_it):
    """What the compute units sustain on loops of nothing but the instructions in question (fmha_pipe_probe of the
    C ABI: two waves on every SIMD of the chip, four matrix instructions per loop trip and wave, 2000 trips), and the
    headline kernel on all-zero operands.  Each entry: TFLOP/s of the 32x32x16 fp16 matrix instructions, the core
    clock the waves saw, and for the mixes the share of the matrix-only rate at the same data.  Diagnostic, never
    part of `value`."""
    res = (C.c_double * 4)()

    def probe(mode, n, rnd, wps=2, iters=2000):
        if L.fmha_pipe_probe(mode, n, rnd, wps, iters, 6, res) != 0:
            return None
        return {"us": round(res[0], 1), "clock_mhz": round(res[1]), "mfma_tflops": round(res[2], 1)}
    out = {"protocol": "fmha_pipe_probe(mode, n, random_data, waves_per_simd=2, iters=2000, launches=6), second half of "
                       "the launches timed between events; MI355X dense fp16 peak 2500 TFLOP/s = one 32x32x16 matrix "
                       "instruction per 32 cycles and SIMD at 2400 MHz"}
    for rnd, tag in ((0, "zero_data"), (1, "random_data")):
        base = probe(1, 2, rnd)
        if base is None:
            return {"unavailable": "fmha_pipe_probe failed"}
        e = {"mfma_only": base, "mfma_only_one_wave_per_simd": probe(1, 2, rnd, wps=1),
             "mfma_one_accumulator_chain": probe(3, 2, rnd)}
        for name, mode, n in (("mfma_plus_2_exp", 2, 2), ("mfma_plus_4_exp", 2, 4), ("mfma_plus_6_exp", 2, 6),
                              ("mfma_plus_softmax_mix_2exp_1cvt_2add", 18, 5),
                              ("mfma_plus_4_v_dot2c_f32_f16", 12, 4), ("mfma_plus_4_v_fma_mix_f32", 19, 4),
                              ("mfma_plus_4_v_xor", 36, 4), ("mfma_plus_8_v_xor", 36, 8),
                              ("mfma_plus_16_v_xor", 36, 16), ("mfma_plus_32_v_xor", 36, 32),
                              ("sibling_waves_one_mfma_one_exp", 4, 4),
                              ("mfma_plus_4_v_cvt_pk_f16_f32", 16, 4), ("mfma_plus_4_v_mad_u64_u32", 20, 4),
                              ("mfma_plus_4_v_bitop3_b32", 21, 4), ("mfma_plus_4_v_mov_b32_dpp", 22, 4),
                              ("mfma_plus_4_v_cndmask_b32", 25, 4), ("mfma_plus_4_v_permlane32_swap", 30, 4)):
            r = probe(mode, n, rnd)
            if r:
                r["share_of_mfma_only"] = round(r["mfma_tflops"] / base["mfma_tflops"], 3)
                # core cycles per group of one matrix instruction and its n vector instructions, per SIMD
                r["cycles_per_group"] = round(r["us"] * r["clock_mhz"] / (2 * 2000 * 4), 1)
            e[name] = r
        v = probe(37, 16, rnd)
        if v:
            v["cycles_per_vector_instruction_per_simd"] = round(v["us"] * v["clock_mhz"] / (2 * 2000 * 4 * 16), 2)
            v.pop("mfma_tflops")
        e["v_xor_only_16_per_group"] = v
        v1 = probe(37, 16, rnd, wps=1)
        if v1:
            v1["cycles_per_vector_instruction_per_simd"] = round(v1["us"] * v1["clock_mhz"] / (2000 * 4 * 16), 2)
            v1.pop("mfma_tflops")
        e["v_xor_only_16_per_group_one_wave_per_simd"] = v1
        out[tag] = e
    # the headline kernel on all-zero q, k, v (same masks): same instruction stream, nothing toggles
    g = torch.Generator().manual_seed(0)
    zs = []
    for _ in range(4):   # as many sets as the headline rotates: the same share of the operands comes from HBM
        z = {n: torch.zeros(B * H, S, D, dtype=torch.float16, device="cuda") for n in ("q", "k", "v")}
        z["o"] = torch.empty_like(z["q"])
        lens = torch.randint(S // 2, S + 1, (B,), generator=g)
        m = torch.zeros(B, 1, 1, S)
        for b in range(B):
            m[b, 0, 0, lens[b]:] = -10000.0
        z["mask"] = m.to(torch.float16).cuda()
        zs.append(z)
    zp = [fwd_params_of(z) for z in zs]
    capi.check(L.fmha_fwd_launch(C.byref(zp[0]), stream))
    ms0 = time_it(lambda i: L.fmha_fwd_launch(C.byref(zp[i % 4]), stream))
    probe_buf = torch.zeros(4, dtype=torch.int64, device="cuda")
    zp[0].clock_probe = probe_buf.data_ptr()
    for i in range(61):
        L.fmha_fwd_launch(C.byref(zp[(i + 3) % 4]), stream)   # ends on set 0
    torch.cuda.synchronize()
    zp[0].clock_probe = None
    c0, t0, c1, t1 = probe_buf.tolist()
    out["headline_kernel_zero_inputs"] = {"us": round(ms0 * 1e3, 2),
                                          "tflops": round(4.0 * B * H * S * S * D / (ms0 * 1e-3) / 1e12, 1),
                                          "effective_core_clock_mhz": round((c1 - c0) / ((t1 - t0) / 100.0), 1) if t1 > t0 else None}
    return out


def cpu_baseline(torch, budget_s=10.0):
    """The CPU baseline on the configuration the reference can run on a CPU: BERT-base attention forward, batch 8,
    heads 12, sequence 128, head dim 64, additive [8,1,1,128] padding mask (valid lengths U{64..128}), the eager
    fp32 composition on the host cores: 3 warm-up calls, then at least 20 timed calls (about 10 s of them)."""
    cores = torch.get_num_threads()
    n, el, flops = _cpu_eager_leg(torch, 8, 12, 128, 64, 64, budget_s, 20)
    return {"value": round(flops * n / el / 1e12, 5), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"B8 H12 S128 D64 fp32, [8,1,1,128] padding mask: 3 warm-up + {n} timed calls of the eager "
                      f"composition (matmul, mask add, softmax, matmul) in {el:.1f} s, torch CPU with {cores} threads",
            "ms_per_iter": round(el / n * 1e3, 4)}


def cpu_headline_sample(torch, budget_s=6.0):
    """The same composition on a bounded sample of the headline workload: 2 of its 32 sequences (32 of the 512
    heads, S 512, D 64, the same kind of padding mask)."""
    cores = torch.get_num_threads()
    n, el, flops = _cpu_eager_leg(torch, 2, H, S, D, S // 2, budget_s, 5)
    return {"value": round(flops * n / el / 1e12, 5), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"{n} timed calls over 2 of the workload's {B} sequences (B2 H{H} S{S} D{D}, padding mask) in "
                      f"{el:.1f} s, torch CPU with {cores} threads",
            "ms_per_iter": round(el / n * 1e3, 4)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--sets", type=int, default=4, help="input sets rotated to defeat the last-level cache")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-bwd", action="store_true", help="skip the train-step (fwd+bwd) leg")
    ap.add_argument("--no-power", action="store_true", help="skip the socket power / clock telemetry leg")
    ap.add_argument("--no-ceilings", action="store_true", help="skip the pipe-ceiling microbenchmarks")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="also run a plain 256 MiB device copy a few times: under `rocprofv3 --pmc FETCH_SIZE` "
                         "(or WRITE_SIZE) its known traffic calibrates the counter for the attention kernels")
    ap.add_argument("--profile", metavar="LEG", default=None,
                    help="run only LEG's launches (fwd, fwd_trim, train, c4, c5, d256, fp8, decode, "
                         "decode_plain) and no "
                         "timing: for rocprofv3 runs in which every dispatch of a kernel is the same workload")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; attention shards over batch*heads without "
              "communication, so N GPUs would each run this same kernel on their slice. Use --gpus 1.",
              file=sys.stderr)
        return 2

    idle_power = None if (args.no_power or args.profile) else smi_sample()  # before this process touches the GPU
    import torch
    from nvfuserexamples_amd import capi
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    L = capi.lib()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)

    if args.traffic_probe:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)   # reads 256 MiB, writes 256 MiB per launch
        torch.cuda.synchronize()
        del src, dst
    if args.profile:
        return profile_leg(torch, capi, L, stream, args)

    # ---- forward (headline): every key tile of the dense shape is visited (FMHA_FLAG_NO_MASK_TRIM), so the
    # flops that are counted are flops that are executed; the library's default (tiles under the hard-masked
    # tail left out, same bits) is `fps` and is timed beside it
    sets = make_inputs(torch, capi, args.sets)
    fps = [fwd_params(capi, t) for t in sets]
    fps_dense = [fwd_params(capi, t, flags=capi.FLAG_NO_MASK_TRIM) for t in sets]
    capi.check(L.fmha_fwd_launch(C.byref(fps[0]), stream))
    capi.check(L.fmha_fwd_launch(C.byref(fps_dense[0]), stream))

    def fwd_step(i):
        if L.fmha_fwd_launch(C.byref(fps[i % len(fps)]), stream):
            raise RuntimeError("forward launch refused inside a timed region")

    def fwd_dense(i):
        if L.fmha_fwd_launch(C.byref(fps_dense[i % len(fps_dense)]), stream):
            raise RuntimeError("forward launch refused inside a timed region")

    spread = {}
    ms, wall_ms = time_steps(torch, fwd_dense, args.steps, args.warmup, stats=spread)
    # effective core clock while the headline kernel runs: counters of its first workgroup, read at the end of
    # another block of the same back-to-back steps right behind the timed ones (clock_probe of the C ABI)
    probe = torch.zeros(4, dtype=torch.int64, device="cuda")
    for i in range(args.steps):
        fwd_dense(i + 1)
    fps_dense[0].clock_probe = probe.data_ptr()
    fwd_dense(0)
    fps_dense[0].clock_probe = None
    torch.cuda.synchronize()
    c0, t0, c1, t1 = probe.tolist()
    eff_clock = round((c1 - c0) / ((t1 - t0) / 100.0), 1) if t1 > t0 else None
    ms_launch = time_launches(torch, fwd_dense, args.steps, args.warmup)
    ms_trim, _ = time_steps(torch, fwd_step, args.steps, args.warmup)
    ms_trim_launch = time_launches(torch, fwd_step, args.steps, args.warmup)
    flops = 4.0 * B * H * S * S * D
    bytes_ = 4.0 * B * H * S * D * 2 + B * S * 2
    tflops = flops / (ms * 1e-3) / 1e12
    # The second headline and the other configurations come next, before the auxiliary legs: those keep the board
    # loaded for tens of seconds, and what is timed behind them runs at the clock of a board that has been hot that long.
    train_part = {}
    # ---- train step (forward with LSE + Philox dropout, then backward): every key tile visited, as the
    # headline; the default (trimming) run and the valid-length run beside it
    if not args.no_bwd:
        tsets = make_inputs(torch, capi, args.sets, seed=1, train=True)
        NT = capi.FLAG_NO_MASK_TRIM
        tf = [fwd_params(capi, t, train=True, flags=NT) for t in tsets]
        tb = [bwd_params(capi, t, flags=NT) for t in tsets]
        rc_f = L.fmha_fwd_launch(C.byref(tf[0]), stream)
        rc_b = L.fmha_bwd_launch(C.byref(tb[0]), stream)
        if rc_f == 0 and rc_b == 0:
            for F in tf:
                L.fmha_fwd_launch(C.byref(F), stream)   # O and LSE of every set, for the backward timed alone

            def train_step(i):
                if L.fmha_fwd_launch(C.byref(tf[i % len(tf)]), stream) or L.fmha_bwd_launch(C.byref(tb[i % len(tb)]), stream):
                    raise RuntimeError("train-step launch refused inside a timed region")

            def bwd_step(i):
                if L.fmha_bwd_launch(C.byref(tb[i % len(tb)]), stream):
                    raise RuntimeError("backward launch refused inside a timed region")

            def fwd_t(i):
                L.fmha_fwd_launch(C.byref(tf[i % len(tf)]), stream)
            tsp = {}
            ms_t, _ = time_steps(torch, train_step, args.steps, args.warmup, stats=tsp)
            ms_b, _ = time_steps(torch, bwd_step, args.steps, args.warmup)
            ms_f, _ = time_steps(torch, fwd_t, args.steps, args.warmup)
            fl_t = 14.0 * B * H * S * S * D
            by_t = 12.0 * B * H * S * D * 2 + 3 * B * H * S * 4 + 2 * B * S * 2
            train_part["fwd_bwd"] = {
                "workload": "same shape, train step: fwd (+LSE) + bwd, Philox dropout p=0.1, padding mask, every key "
                            "tile visited (FMHA_FLAG_NO_MASK_TRIM)",
                "ms_per_step": round(ms_t, 5), "tflops": round(fl_t / (ms_t * 1e-3) / 1e12, 2),
                "frac_of_mfma_peak": round(fl_t / (ms_t * 1e-3) / 1e12 / PEAK_MFMA_TFLOPS, 4),
                "hbm_frac": round(by_t / (ms_t * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4),
                "fwd_only_ms": round(ms_f, 5), "bwd_only_ms": round(ms_b, 5),
                "bwd_only_tflops": round(10.0 * B * H * S * S * D / (ms_b * 1e-3) / 1e12, 2),
                "timing": tsp}
            for P in tf + tb:
                P.flags = 0
            ms_tt, _ = time_steps(torch, train_step, args.steps, args.warmup)
            ms_bt, _ = time_steps(torch, bwd_step, args.steps, args.warmup)
            tlens = [(t["mask"][:, 0, 0, :] == 0).sum(dim=1).to(torch.int32).contiguous() for t in tsets]
            vis_t = float(sum(((n.float() / 128).ceil() * 128 / S).mean().item() for n in tlens) / len(tlens))
            train_part["fwd_bwd"].update(mask_trim_ms_per_step=round(ms_tt, 5), mask_trim_bwd_only_ms=round(ms_bt, 5),
                                  mask_trim_tflops_dense_count=round(fl_t / (ms_tt * 1e-3) / 1e12, 2),
                                  mask_trim_visited_tile_share=round(vis_t, 4),
                                  mask_trim_tflops_executed=round(fl_t * vis_t / (ms_tt * 1e-3) / 1e12, 2))
            # the same train step with the valid lengths handed over as counts (kv_len) instead of the mask
            # tensor: same results, key tiles past a sequence's length skipped in all three kernels
            for P, n in zip(tf + tb, tlens + tlens):
                P.mask, P.mask_kind = None, capi.MASK_NONE
                P.kv_len, P.kv_len_bh_div = n.data_ptr(), H
            if L.fmha_fwd_launch(C.byref(tf[0]), stream) == 0 and L.fmha_bwd_launch(C.byref(tb[0]), stream) == 0:
                ms_tl, _ = time_steps(torch, train_step, args.steps, args.warmup)
                train_part["fwd_bwd"]["kv_len_ms_per_step"] = round(ms_tl, 5)
                train_part["fwd_bwd"]["kv_len_speedup_vs_default_mask_path"] = round(ms_tt / ms_tl, 3)
        else:
            train_part["fwd_bwd"] = {"error": f"fwd rc={rc_f} bwd rc={rc_b}: " + L.fmha_strerror(rc_b or rc_f).decode()}
        del tsets
        torch.cuda.empty_cache()
        # ---- the other train-step configurations (no padding): long sequences, and wide heads in bf16 under the causal mask
        train_part["configs"] = {
            "C4_long_sequence": config_leg(torch, capi, L, stream, args.steps, args.warmup, 4, 16, 2048, 64, "f16",
                                           False, 0.1, 1.0, 2),
            "C5_wide_head_bf16_causal": config_leg(torch, capi, L, stream, args.steps, args.warmup, 16, 32, 1024, 128,
                                                   "bf16", True, 0.0, 0.5, 1),
        }

    # warm-cache figure for reference: one input set only
    def fwd_warm(i):
        L.fmha_fwd_launch(C.byref(fps_dense[0]), stream)
    ms_warm, _ = time_steps(torch, fwd_warm, args.steps, args.warmup)
    # the same steps dealt to two streams in turn (default priority): the first workgroups of a launch start
    # on the compute units that the previous launch has already left, which hides the drain-and-dispatch
    # gap between back-to-back launches on one stream.  Reported beside the headline, never as `value`.
    s2 = [torch.cuda.Stream(), torch.cuda.Stream()]
    s2p = [C.c_void_p(x.cuda_stream) for x in s2]
    def two_stream_steps(n):
        for i in range(n):
            L.fmha_fwd_launch(C.byref(fps[i % len(fps)]), s2p[i & 1])
    torch.cuda.synchronize()
    two_stream_steps(max(args.warmup, 2000))
    torch.cuda.synchronize()
    regions = []
    for _ in range(BLOCKS):
        t0 = time.perf_counter()
        two_stream_steps(max(args.steps, 100))
        torch.cuda.synchronize()
        regions.append((time.perf_counter() - t0) * 1e3 / max(args.steps, 100))  # host clock, synchronised both ends
    ms_two = _median(regions)
    tflops_launch = flops / (ms_launch * 1e-3) / 1e12
    # the same batches with the valid lengths handed over as counts (kv_len) instead of an additive
    # mask: same outputs bit for bit, key tiles past a sequence's length are skipped.  Reported
    # beside the headline, never as `value` (the reference's operators take the mask tensor).
    lens = [(t["mask"][:, 0, 0, :] == 0).sum(dim=1).to(torch.int32).contiguous() for t in sets]
    lps = []
    for t, n in zip(sets, lens):
        P = fwd_params(capi, t)
        P.mask, P.mask_kind = None, capi.MASK_NONE
        P.kv_len, P.kv_len_bh_div = n.data_ptr(), H
        lps.append(P)
    def fwd_len(i):
        L.fmha_fwd_launch(C.byref(lps[i % len(lps)]), stream)
    capi.check(L.fmha_fwd_launch(C.byref(lps[0]), stream))
    ms_len, _ = time_steps(torch, fwd_len, args.steps, args.warmup)
    # the same batches kept as a packed [B,S,3,H,D] projection output, read in place, with O written
    # as [B,S,H,D]: what a caller gets who does not permute into the folded layout first.  Reported
    # beside the headline, never as `value` (the reference's operators take folded tensors); the
    # permute copies it spares (three in, one out) are timed beside it.
    pks, pps = [], []
    for t, fp in zip(sets, fps):
        pk = torch.empty(B, S, 3, H, D, dtype=torch.float16, device="cuda")
        for j, n in enumerate(("q", "k", "v")):
            pk[:, :, j] = t[n].view(B, H, S, D).permute(0, 2, 1, 3)
        o4 = torch.empty(B, S, H, D, dtype=torch.float16, device="cuda")
        P = fwd_params(capi, t)
        P.q, P.k, P.v = (pk[:, :, j].data_ptr() for j in range(3))
        P.o, P.heads = o4.data_ptr(), H
        for name in ("q_stride", "k_stride", "v_stride"):
            getattr(P, name)[:] = [S * 3 * H * D, D, 3 * H * D]
        P.o_stride[:] = [S * H * D, D, H * D]
        pks.append((pk, o4))
        pps.append(P)
    def fwd_packed(i):
        L.fmha_fwd_launch(C.byref(pps[i % len(pps)]), stream)
    capi.check(L.fmha_fwd_launch(C.byref(pps[0]), stream))
    ms_packed, _ = time_steps(torch, fwd_packed, args.steps, args.warmup)
    def permutes(i):
        pk, o4 = pks[i % len(pks)]
        for j in range(3):
            pk[:, :, j].permute(0, 2, 1, 3).contiguous()
        o4.permute(0, 2, 1, 3).contiguous()
    ms_perm, _ = time_steps(torch, permutes, max(10, args.steps // 4), 5)
    del pks, pps
    power = None if args.no_power else power_probe(torch, fwd_dense, idle_power)
    ceilings = None
    if not args.no_ceilings:
        ceilings = pipe_ceilings(torch, capi, L, stream,
                                 lambda t: fwd_params(capi, t, flags=capi.FLAG_NO_MASK_TRIM),
                                 lambda step: time_steps(torch, step, args.steps, args.warmup)[0])
        ceilings["headline_kernel_random_inputs"] = {"us": round(ms * 1e3, 2), "tflops": round(tflops, 1),
                                                     "effective_core_clock_mhz": eff_clock}
    # share of the (query tile, 128-key tile pair) products the kernel really visits: it leaves out the tile
    # pairs that hold only hard-masked keys (their weights are exactly zero)
    visited = float(sum(((n.float() / 128).ceil() * 128 / S).mean().item() for n in lens) / len(lens))
    del sets, fps, fps_dense, lps, lens

    traffic_bytes, traffic_commit = measured_traffic("fmha_fwd_head_kernel_B32H16S512D64_f16")
    out = {
        "metric": "MHA fwd TFLOP/s (B32,H16,S512,D64 fp16)", "value": round(tflops, 2), "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "BERT-large attention forward: B32 H16 S512 D64 fp16, additive [B,1,1,S] "
                               "padding mask (valid length U{256..512}), scale 1/8, no dropout; every key tile "
                               "visited (FMHA_FLAG_NO_MASK_TRIM)",
                   "layout": "[B*H,S,D] contiguous", "input_sets_rotated": args.sets},
        "timing": dict(spread, protocol=f"{args.warmup} warm-up steps + {BURN_S} s of the same steps, then the median of "
                                        f"{BLOCKS} blocks of {args.steps} steps, each between HIP events and a synchronisation"),
        "value_frac_of_mfma_peak": round(tflops / PEAK_MFMA_TFLOPS, 4),
        # achieved = algorithmic flops of one launch / launch duration (event pair per launch, median block);
        # traffic = HBM bytes per launch from rocprofv3 FETCH_SIZE + WRITE_SIZE, each scaled by what the
        # counter reads for a 256 MiB copy (profiles/traffic.json, profiles/fmha_fwd_head_kernel_B32H16S512D64_f16.md)
        "roofline": {"bound": "mfma", "achieved": round(tflops_launch, 2), "peak": PEAK_MFMA_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(tflops_launch / PEAK_MFMA_TFLOPS, 4),
                     "traffic": traffic_bytes, "traffic_from_commit": traffic_commit,
                     "kernel": HEADLINE_KERNEL, "flops_per_launch": flops,
                     "executed_frac": round(tflops_launch / PEAK_MFMA_TFLOPS, 4),   # every counted tile is visited
                     "visited_tile_share": 1.0,
                     "algorithmic_bytes_per_launch": bytes_,
                     "hbm_achieved_GBps": round(bytes_ / (ms * 1e-3) / 1e9, 1),
                     "hbm_frac": round(bytes_ / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4),
                     "hbm_achieved_GBps_launch": round(bytes_ / (ms_launch * 1e-3) / 1e9, 1),
                     "launch_us": round(ms_launch * 1e3, 2),
                     "launch_gap_us": round((ms - ms_launch) * 1e3, 2)},
        # the library's default on the same batches: key tiles that hold only hard-masked keys are left out
        # (bit-identical outputs); flops still counted for the dense shape, and the share really executed
        "fwd_mask_trim": {"ms_per_step": round(ms_trim, 5), "launch_us": round(ms_trim_launch * 1e3, 2),
                          "tflops_dense_count": round(flops / (ms_trim * 1e-3) / 1e12, 2),
                          "visited_tile_share": round(visited, 4),
                          "tflops_executed": round(flops * visited / (ms_trim * 1e-3) / 1e12, 2),
                          "speedup_vs_every_tile": round(ms / ms_trim, 3)},
        "fwd_warm_cache": {"ms_per_step": round(ms_warm, 5),
                           "tflops": round(flops / (ms_warm * 1e-3) / 1e12, 2)},
        "host_wall_ms_per_step": round(wall_ms, 5),
        "fwd_two_streams": {"workload": "the default steps issued to two streams in turn (independent batches in flight "
                                        "together); host clock over the whole region",
                            "ms_per_step": round(ms_two, 5), "speedup_vs_one_stream": round(ms_trim / ms_two, 3)},
        "fwd_kv_len": {"workload": "same batches, valid lengths passed as counts instead of the mask tensor",
                       "ms_per_step": round(ms_len, 5), "speedup_vs_default_mask_path": round(ms_trim / ms_len, 3)},
        "fwd_packed_qkv": {"workload": "same batches as a packed [B,S,3,H,D] tensor read in place, O written as "
                                       "[B,S,H,D] (default mask path)",
                           "ms_per_step": round(ms_packed, 5),
                           "permute_copies_spared_ms": round(ms_perm, 5)},
    }

    out.update(train_part)
    out["short_sequences"] = short_sequence_legs(torch, capi, L, stream, args.steps, args.warmup)
    out["operators_BH512_S128_D64"] = operator_legs(torch, args.steps, args.warmup)
    out["torch_sdpa_same_gpu"] = torch_sdpa_context(torch, args.steps, args.warmup)
    out["head_dim_256"] = head_dim_256_leg(torch, capi)
    out["fp8_e4m3_forward"] = fp8_leg(torch, capi, L, stream, args.steps, args.warmup)
    out["decode_steps"] = decode_leg(torch, capi, args.steps, args.warmup)
    out["power"] = power
    out["pipe_ceilings"] = ceilings
    out["effective_core_clock_mhz"] = eff_clock  # MFMA peak is quoted at the maximum clock (2400 MHz)

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(torch)
        out["cpu_baseline_headline_sample"] = cpu_headline_sample(torch)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
