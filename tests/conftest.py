import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def has_gpu():
    import torch
    return torch.cuda.is_available()


def make_qkv(bh, sq, sk, d, seed=0, std=1.0, dtype="fp16", with_dout=False):
    """Seeded inputs, generated in fp32 on the CPU and rounded to the element type so the
    CPU oracle and the GPU see identical bits.  Returns torch CPU tensors of that type."""
    import torch
    g = torch.Generator().manual_seed(seed)
    tdt = {"fp16": torch.float16, "bf16": torch.bfloat16}[dtype]
    out = [(torch.randn(bh, s, d, generator=g) * std).to(tdt) for s in (sq, sk, sk)]
    if with_dout:
        out.append((torch.randn(bh, sq, d, generator=g) * std).to(tdt))
    return out


def pad_mask(b, sk, lo, hi, seed=0, neg=-10000.0):
    """[B,1,1,sk] additive padding mask: 0 on the first L keys, `neg` after, L ~ U{lo..hi}."""
    import torch
    g = torch.Generator().manual_seed(seed + 1000)
    lens = torch.randint(lo, hi + 1, (b,), generator=g)
    m = torch.zeros(b, 1, 1, sk)
    for i in range(b):
        m[i, 0, 0, lens[i]:] = neg
    return m


def tail_mask(kind, b, sk, seed):
    """[B,1,1,sk] additive masks with a (mostly hard-masked) tail per row, for the tests of key tiles
    that are skipped because the mask leaves nothing in them."""
    import torch
    g = torch.Generator().manual_seed(seed)
    m = torch.zeros(b, 1, 1, sk)
    lens = torch.randint(1, sk + 1, (b,), generator=g)
    for i in range(b):
        n = int(lens[i])
        if kind == "tail":
            m[i, ..., n:] = -10000.0
        elif kind == "inf":
            m[i, ..., n:] = float("-inf")
        elif kind == "holes":                       # masked keys inside the live range as well
            m[i, ..., n:] = -10000.0
            m[i, 0, 0, torch.rand(sk, generator=g) < 0.3] = -10000.0
        elif kind == "soft":                        # a tail that is NOT hard: nothing may be skipped
            m[i, ..., n:] = -100.0
        elif kind == "last_live":                   # only the very last key is visible
            m[i, ..., : sk - 1] = -10000.0
        elif kind == "some_rows_all_masked":        # a fully masked row is a softmax over all keys
            m[i] = -10000.0 if i % 2 else 0.0
            if not i % 2:
                m[i, ..., n:] = -10000.0
    return m


def f32(t):
    return t.float().numpy()


def rel_to_max(a, b, floor=1e-30):
    """max |a-b| relative to max |b|; `floor` keeps exactly-zero answers (e.g. the gradient of a
    one-key softmax) from turning rounding dust into an infinite ratio."""
    return float(np.abs(a - b).max() / max(np.abs(b).max(), floor))
