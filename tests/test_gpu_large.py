"""Tensors of more than 2^31 elements (a 288 GB card invites them): every offset into q, k, v, o and the
gradients must be formed in 64 bits.  No CPU answer at this size; instead heads from the beginning, the middle
and the very end of the big problem are recomputed alone (small tensors, offsets far below 2^31) and must come
out bit for bit the same -- the kernels are deterministic and treat heads independently."""
import pytest
import torch

from nvfuserexamples_amd import capi

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype,causal", [(torch.float16, False), (torch.bfloat16, True)])
def test_offsets_beyond_32_bits(dtype, causal):
    bh, s, d, h = 36000, 1024, 64, 16          # 2.36e9 elements per tensor
    assert bh * s * d > 2 ** 31
    free, _ = torch.cuda.mem_get_info()
    if free < 60 * 2 ** 30:
        pytest.skip("needs about 45 GB of device memory")
    g = torch.Generator(device="cuda").manual_seed(3)
    q, k, v, do = (torch.randn(bh, s, d, device="cuda", dtype=dtype, generator=g) for _ in range(4))
    m = None
    if not causal:
        lens = torch.randint(s // 2, s + 1, (bh // h,), device="cuda", generator=g)
        m = torch.zeros(bh // h, 1, 1, s, device="cuda", dtype=dtype)
        m.masked_fill_(torch.arange(s, device="cuda").view(1, 1, 1, s) >= lens.view(-1, 1, 1, 1), -10000.0)
    o, lse, _, _ = capi.fwd(q, k, v, mask=m, causal=causal, want_lse=True)
    dq, dk, dv = capi.bwd(do, q, k, v, o, lse, mask=m, causal=causal)
    torch.cuda.synchronize()
    for lo in (0, (bh // 2 // h) * h, bh - h):             # whole sequences: their heads share a mask row
        sl = slice(lo, lo + h)
        ms = None if m is None else m[lo // h:lo // h + 1].contiguous()
        qs, ks, vs, ds = (t[sl].contiguous() for t in (q, k, v, do))
        o1, l1, _, _ = capi.fwd(qs, ks, vs, mask=ms, causal=causal, want_lse=True)
        g1 = capi.bwd(ds, qs, ks, vs, o1, l1, mask=ms, causal=causal)
        torch.cuda.synchronize()
        assert torch.equal(o1, o[sl]) and torch.equal(l1, lse[sl]), lo
        for a, b in zip(g1, (dq, dk, dv)):
            assert torch.equal(a, b[sl]), lo
