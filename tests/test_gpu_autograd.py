"""loss.backward() through the autograd wrapper matches autograd through the eager composition
(fp32, same keep decisions) to the gradient bar of the backward tests."""
import numpy as np
import pytest
import torch

import oracle
from oracle import eager
from conftest import make_qkv, pad_mask

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("causal,p", [(False, 0.0), (True, 0.1)])
def test_autograd_wrapper_matches_eager_autograd(causal, p):
    from nvfuserexamples_amd.autograd import attention
    bh, s, d = 8, 192, 64
    q, k, v, do = (t.cuda() for t in make_qkv(bh, s, s, d, seed=5, with_dout=True))
    m = pad_mask(4, s, s // 2, s).half().cuda()
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    o = attention(qa, ka, va, mask=m, is_causal=causal, p_drop=p, seed=11, offset=2)
    (o.float() * do.float()).sum().backward()

    keep = None
    if p > 0:
        keep = torch.from_numpy(oracle.keep_mask(11, 2, p, bh, s, s).astype(np.float32)).cuda()
    qe, ke, ve = (t.float().clone().requires_grad_(True) for t in (q, k, v))
    add = m.float().expand(4, 2, 1, s).reshape(bh, 1, s)
    s_ = qe.matmul(ke.transpose(1, 2)) * d ** -0.5 + add
    if causal:
        s_ = s_.masked_fill(~torch.ones(s, s, dtype=torch.bool, device="cuda").tril(), float("-inf"))
    pr = torch.softmax(s_, -1)
    if keep is not None:
        pr = pr * keep * oracle.drop_scale(p)   # the mean-preserving factor at the realised keep probability
    oe = pr.matmul(ve)
    (oe * do.float()).sum().backward()
    assert (o.float() - oe).abs().max().item() <= 2e-3
    for a, b in ((qa.grad, qe.grad), (ka.grad, ke.grad), (va.grad, ve.grad)):
        assert (a.float() - b).abs().max().item() <= 1e-2 * b.abs().max().item()


def test_the_operator_itself_is_differentiable():
    """torch.ops.mha_manual.fmha_fwd carries its autograd formula in C++ (Autograd dispatch key): no Python
    wrapper is needed, the row log-sum-exp is marked non-differentiable, and under no_grad nothing is recorded."""
    from nvfuserexamples_amd import load_ops
    from nvfuserexamples_amd import capi
    ops = load_ops()
    bh, s, d = 4, 160, 64
    q, k, v, do = (t.cuda() for t in make_qkv(bh, s, s, d, seed=9, with_dout=True))
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    o, lse = ops.fmha_fwd(qa, ka, va, None, 0.0, True, 0.1, 3, 1)
    assert o.requires_grad and not lse.requires_grad
    o.backward(do)
    dq, dk, dv = capi.bwd(do, q, k, v, o.detach(), lse, causal=True, drop_kind=capi.DROP_PHILOX, p_drop=0.1, seed=3, offset=1)
    torch.cuda.synchronize()
    assert torch.equal(qa.grad, dq) and torch.equal(ka.grad, dk) and torch.equal(va.grad, dv)
    with torch.no_grad():
        o2, _ = ops.fmha_fwd(qa, ka, va, None, 0.0, True, 0.1, 3, 1)
    assert not o2.requires_grad and torch.equal(o2, o.detach())
