"""Writes the committed golden vectors from the CPU oracle (run from the repo root:
``python tests/golden/make_fixtures.py``).  Inputs are seeded and already rounded to fp16."""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))
import oracle  # noqa: E402
from conftest import make_qkv, pad_mask  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    bh, sq, sk, d = 2, 64, 128, 64
    q, k, v, do = make_qkv(bh, sq, sk, d, seed=42, with_dout=True)
    m = pad_mask(1, sk, sk // 2, sk, seed=42).half()
    seed, offset, p = 0x1234, 7, 0.1
    kw = dict(mask=m.float().numpy(), philox=True, p_drop=p, seed=seed, offset=offset)
    r = oracle.attention(q.float().numpy(), k.float().numpy(), v.float().numpy(), dout=do.float().numpy(),
                         want=("o", "lse", "dq", "dk", "dv"), **kw)
    np.savez_compressed(os.path.join(HERE, "fwd_small.npz"),
                        q=q.numpy(), k=k.numpy(), v=v.numpy(), dout=do.numpy(), mask=m.numpy(),
                        seed=seed, offset=offset, p_drop=p, **{n: a for n, a in r.items()})
    # Philox keep decisions for a fixed (seed, offset): 1 bit per element
    km = oracle.keep_mask(seed, offset, p, 2, 40, 52)
    np.savez_compressed(os.path.join(HERE, "keep_mask.npz"), keep=np.packbits(km), shape=km.shape,
                        seed=seed, offset=offset, p_drop=p)


if __name__ == "__main__":
    main()
