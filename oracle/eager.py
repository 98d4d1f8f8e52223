"""Eager torch restatement of the reference's ground-truth compositions.

TEST INFRASTRUCTURE ONLY (same rule as the rest of ``oracle/``).  These are the
library-routine compositions (matmul, softmax) the reference itself compares
its fused kernels against; they pin the C restatement and serve as the CPU
baseline timed by the benchmark.
"""
import torch


def infer_mha(q, k, v, amask, neg=-10000.0, scale=None):
    """Inference composition in fp32 (reference test.py:12-18): 0/1 mask -> (1-m)*neg."""
    scale = q.shape[-1] ** -0.5 if scale is None else scale
    s = q.float().matmul(k.float().transpose(1, 2)) * scale
    s = s + (1.0 - amask.float()) * neg
    p = torch.softmax(s, -1)
    return p.matmul(v.float())


def train_mha(q, k, v, pad_mask, dropout_mask, keep_prob=0.5, scale=None, dtype=torch.float32):
    """Train composition (reference test_train_mha.py:14-21): returns (softmax, dropped, ctx).

    The reference divides by its ``dropout_prob`` constant, i.e. treats it as
    the keep probability; ``keep_prob`` keeps that meaning.
    """
    scale = q.shape[-1] ** -0.5 if scale is None else scale
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    s = q.matmul(k.transpose(1, 2)) * scale + pad_mask.to(dtype)
    p = torch.softmax(s, -1)
    pd = (p / keep_prob) * dropout_mask.to(dtype)
    return p, pd, pd.matmul(v)


def general_mha(q, k, v, add_mask=None, causal=False, scale=None, keep=None, drop_scale=1.0,
                dtype=torch.float32):
    """General additive-mask / causal / keep-mask composition; differentiable."""
    scale = q.shape[-1] ** -0.5 if scale is None else scale
    s = q.to(dtype).matmul(k.to(dtype).transpose(1, 2)) * scale
    if add_mask is not None:
        s = s + add_mask.to(dtype)
    if causal:
        sq, sk = s.shape[-2:]
        tri = torch.ones(sq, sk, dtype=torch.bool).tril()
        s = s.masked_fill(~tri, float("-inf"))
    p = torch.softmax(s, -1)
    if keep is not None:
        p = p * keep.to(dtype) * drop_scale
    return p.matmul(v.to(dtype))
