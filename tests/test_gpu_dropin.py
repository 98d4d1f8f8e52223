"""The reference's own test flows, through torch.ops.mha_manual, at the reference's shapes.

test.py:20-29 and test_train_mha.py:23-41 build unseeded random half inputs of shape
[512,128,64] with full [512,128,128] 0/1 masks, call the fused op and assert
torch.allclose(atol=1e-2) against an eager composition.  Same calls here, seeded, with the
reference's bound and this build's tighter one."""
import pytest
import torch

from oracle import eager

pytestmark = pytest.mark.gpu

BH, S, D = 32 * 16, 128, 64


@pytest.fixture(scope="module")
def ops():
    import mha_manual  # noqa: F401
    return torch.ops.mha_manual


def _inputs(seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    q, k, v = (torch.randn((BH, S, D), dtype=torch.half, device="cuda", generator=g) for _ in range(3))
    m1 = torch.empty((BH, S, S), device="cuda").random_(2, generator=g).to(torch.half)
    m2 = torch.empty((BH, S, S), device="cuda").random_(2, generator=g).to(torch.half)
    return q, k, v, m1, m2


def test_inference_op_like_reference_test(ops):
    q, k, v, amask, _ = _inputs(0)
    fused = ops.fmha_nvfuser(q, k, v, amask)
    ctx = eager.infer_mha(q, k, v, amask).to(torch.half)   # fp32 eager on the GPU, as test.py:12-18
    assert fused.dtype == torch.half and fused.shape == q.shape
    assert torch.allclose(ctx, fused, atol=1e-2)
    assert (ctx.float() - fused.float()).abs().max().item() <= 2e-3


def test_train_ops_like_reference_test(ops):
    q, k, v, pm, dm = _inputs(1)
    pad_mask = pm * (-1000)
    sm_ref, dr_ref, ctx = eager.train_mha(q, k, v, pad_mask, dm, keep_prob=0.5)   # fp32 eager
    fused = ops.fmha_train_nvfuser(q, k, v, pad_mask, dm)
    saved = ops.fmha_train_saveim_nvfuser(q, k, v, pad_mask, dm)
    assert isinstance(saved, (list, tuple)) and len(saved) == 3
    assert torch.allclose(fused, ctx.half(), atol=1e-2)
    assert torch.allclose(saved[0], ctx.half(), atol=1e-2)
    assert torch.equal(saved[0], fused)
    assert (saved[1].float() - sm_ref).abs().max().item() <= 1e-3
    assert (saved[2].float() - dr_ref).abs().max().item() <= 2e-3


def test_inference_op_at_a_narrower_head(ops):
    """The reference's operator exists at head dim 64 only (fmha/fmha_manual.cpp:24-29); here narrower rows of
    whole 16-byte pieces run as they are, scaled by 1/sqrt(d): the reference's 1/8 (fmha/fmha_manual.cpp:68) at d = 64."""
    q, k, v, amask, _ = _inputs(5)
    q, k, v = (t[:, :, :48].contiguous() for t in (q, k, v))
    fused = ops.fmha_nvfuser(q, k, v, amask)
    ctx = eager.infer_mha(q, k, v, amask)
    assert fused.shape == q.shape
    assert (ctx.float() - fused.float()).abs().max().item() <= 2e-3


def test_general_ops_roundtrip(ops):
    q, k, v, _, _ = _inputs(2)
    o, lse = ops.fmha_fwd(q, k, v, None, 0.0, False, 0.0, 0, 0)
    ref = eager.general_mha(q, k, v)
    assert (o.float() - ref).abs().max().item() <= 2e-3
    assert lse.shape == (BH, S) and lse.dtype == torch.float32
    km = ops.fmha_philox_keep_mask(q, 4, S, S, 0.1, 3, 4)
    assert km.dtype == torch.uint8 and abs(km.float().mean().item() - (1 - 26 / 256)) < 5e-3


def test_errors_surface_as_runtime_errors(ops):
    q, k, v, m, _ = _inputs(3)
    with pytest.raises(RuntimeError):   # rows must be whole 16-byte pieces
        ops.fmha_nvfuser(q[:, :, :44].contiguous(), k[:, :, :44].contiguous(), v[:, :, :44].contiguous(), m)
    with pytest.raises(RuntimeError):
        ops.fmha_nvfuser(q, k, v, m[:, :, :64])
    with pytest.raises(RuntimeError):
        ops.fmha_nvfuser(q.float(), k.float(), v.float(), m.float())
