"""Differentiable attention: a thin front to ``torch.ops.mha_manual.fmha_fwd``.

The reference registers its operators without an autograd formula (reference
fmha/fmha_manual.cpp:1240-1250: no Autograd key, its perf runs are under ``no_grad``).  Here
``fmha_fwd`` carries one, registered in C++ under the Autograd dispatch key (fmha/fmha_manual.cpp,
``FmhaFunction``): its backward calls ``fmha_bwd`` with the saved q, k, v, O and row log-sum-exp.
Dropout decisions are never stored: the backward regenerates them from the same ``(seed, offset)``.
"""
from . import load_ops


def attention(q, k, v, mask=None, scale=0.0, is_causal=False, p_drop=0.0, seed=0, offset=0, kv_len=None):
    """softmax(scale * q k^T + mask [causal]) with Philox dropout, times v.

    q ``[B*H,Sq,D]``, k/v ``[B*H,Sk,D]`` contiguous, or 4-d ``[B,H,S,D]`` views of any batch / head /
    row strides (``x.view(B,S,H,D).transpose(1,2)``, slices of a packed QKV projection), read in
    place; fp16 or bf16, on the GPU.  ``mask`` additive, shaped ``[B*H,Sq,Sk]``, ``[B*H,1,Sk]`` or
    ``[B,1,1,Sk]``; ``scale <= 0`` means ``1/sqrt(D)``.
    ``kv_len``: optional int32 GPU vector of B valid key counts (B divides B*H): keys at or past a
    head's count are excluded and their key tiles skipped.  Masks and counts receive no gradient."""
    return load_ops().fmha_fwd(q, k, v, mask, float(scale), bool(is_causal), float(p_drop), int(seed), int(offset),
                               kv_len)[0]
