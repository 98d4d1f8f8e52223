"""The C ABI from several host threads at once.

The reference compiles its kernels lazily behind an unsynchronised "compiled yet?" check and keeps
them in process-global singletons (fmha/fmha_manual.cpp:409,807,1214): not safe to call from two
threads.  This library is stateless apart from per-kernel attributes set once behind thread-safe
statics, so concurrent callers on their own streams must all get the serial answers, bit for bit.
(Run alone, `pytest tests/test_gpu_threads.py`, these are also the first calls of the process, which
is where the one-time set-up would race.)
"""
import threading

import pytest
import torch

from nvfuserexamples_amd import capi
from conftest import make_qkv

pytestmark = pytest.mark.gpu

SHAPES = [
    # bh, sq, sk, d, causal, p_drop     (different kernels: short / general backward, both head dims)
    (6, 128, 128, 64, False, 0.1),
    (4, 320, 320, 64, True, 0.0),
    (2, 256, 384, 128, False, 0.0),
    (3, 200, 200, 64, True, 0.2),
]


def _train_step(t, causal, p):
    q, k, v, do = t
    kw = dict(causal=causal)
    if p:
        kw.update(drop_kind=capi.DROP_PHILOX, p_drop=p, seed=3, offset=9)
    o, lse, _, _ = capi.fwd(q, k, v, want_lse=True, **kw)
    return (o, lse) + tuple(capi.bwd(do, q, k, v, o, lse, **kw))


def test_concurrent_callers_get_the_serial_answers():
    inputs = [[x.cuda() for x in make_qkv(bh, sq, sk, d, seed=i, std=0.5 if d == 128 else 1.0, with_dout=True)]
              for i, (bh, sq, sk, d, _, _) in enumerate(SHAPES)]
    results = [None] * len(SHAPES)
    errors = []
    start = threading.Barrier(len(SHAPES))

    def worker(i):
        try:
            stream = torch.cuda.Stream()   # default priority
            stream.wait_stream(torch.cuda.default_stream())
            start.wait()
            with torch.cuda.stream(stream):
                for _ in range(10):
                    out = _train_step(inputs[i], SHAPES[i][4], SHAPES[i][5])
                stream.synchronize()
            results[i] = out
        except Exception as e:  # surfaced below: an assertion in a thread would otherwise be lost
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(SHAPES))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    torch.cuda.synchronize()
    for i, (_, _, _, _, causal, p) in enumerate(SHAPES):
        want = _train_step(inputs[i], causal, p)
        torch.cuda.synchronize()
        for a, b in zip(results[i], want):
            assert torch.equal(a, b), i
