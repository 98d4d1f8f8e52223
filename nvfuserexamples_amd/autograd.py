"""Differentiable attention on top of ``torch.ops.mha_manual.fmha_fwd`` / ``fmha_bwd``.

The reference registers its operators without an autograd formula
(reference fmha/fmha_manual.cpp:1240-1250: no Autograd key, perf runs under ``no_grad``);
this wrapper ties the forward and backward kernels of this build together so that
``loss.backward()`` works.  Dropout decisions are never stored: the backward regenerates
them from the same ``(seed, offset)``.
"""
import torch

from . import load_ops


class _Attention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, mask, scale, is_causal, p_drop, seed, offset, kv_len):
        ops = load_ops()
        o, lse = ops.fmha_fwd(q, k, v, mask, scale, is_causal, p_drop, seed, offset, kv_len)
        ctx.save_for_backward(q, k, v, o, lse, mask if mask is not None else q.new_empty(0),
                              kv_len if kv_len is not None else q.new_empty(0, dtype=torch.int32))
        ctx.has_mask = mask is not None
        ctx.has_len = kv_len is not None
        ctx.args = (scale, is_causal, p_drop, seed, offset)
        return o

    @staticmethod
    def backward(ctx, dout):
        q, k, v, o, lse, mask, kv_len = ctx.saved_tensors
        scale, is_causal, p_drop, seed, offset = ctx.args
        ops = load_ops()
        dq, dk, dv = ops.fmha_bwd(dout, q, k, v, o, lse, mask if ctx.has_mask else None,
                                  scale, is_causal, p_drop, seed, offset, kv_len if ctx.has_len else None)
        return dq, dk, dv, None, None, None, None, None, None, None


def attention(q, k, v, mask=None, scale=0.0, is_causal=False, p_drop=0.0, seed=0, offset=0, kv_len=None):
    """softmax(scale * q k^T + mask [causal]) with Philox dropout, times v.

    q ``[B*H,Sq,D]``, k/v ``[B*H,Sk,D]`` contiguous, or 4-d ``[B,H,S,D]`` views of any batch / head /
    row strides (``x.view(B,S,H,D).transpose(1,2)``, slices of a packed QKV projection), read in
    place; fp16 or bf16, on the GPU.  ``mask`` additive, shaped ``[B*H,Sq,Sk]``, ``[B*H,1,Sk]`` or
    ``[B,1,1,Sk]``; ``scale <= 0`` means ``1/sqrt(D)``.
    ``kv_len``: optional int32 GPU vector of B valid key counts (B divides B*H): keys at or past a
    head's count are excluded and their key tiles skipped.  Masks and counts receive no gradient."""
    return _Attention.apply(q, k, v, mask, float(scale), bool(is_causal), float(p_drop), int(seed), int(offset),
                            kv_len)
