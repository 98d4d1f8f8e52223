"""The committed golden vectors stay consistent with the oracle (no GPU needed)."""
import os

import numpy as np

import oracle

HERE = os.path.join(os.path.dirname(__file__), "golden")


def test_forward_backward_fixture_matches_oracle():
    f = np.load(os.path.join(HERE, "fwd_small.npz"))
    p = float(f["p_drop"])
    r = oracle.attention(f["q"].astype(np.float32), f["k"].astype(np.float32), f["v"].astype(np.float32),
                         mask=f["mask"].astype(np.float32), philox=True, p_drop=p,
                         seed=int(f["seed"]), offset=int(f["offset"]), dout=f["dout"].astype(np.float32),
                         want=("o", "lse", "dq", "dk", "dv"))
    for n, a in r.items():
        assert np.array_equal(a, f[n]), n


def test_keep_mask_fixture_matches_oracle():
    f = np.load(os.path.join(HERE, "keep_mask.npz"))
    shape = tuple(int(x) for x in f["shape"])
    km = oracle.keep_mask(int(f["seed"]), int(f["offset"]), float(f["p_drop"]), *shape)
    assert np.array_equal(np.packbits(km), f["keep"])
