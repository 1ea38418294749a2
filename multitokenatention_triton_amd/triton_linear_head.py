"""Head-axis linear ("head mixing") operator (HIP-backed).

Mirrors TritonLinearHead (triton_linear_head.py:373-401) and TritonLinearHeadFunction
(:281-370) of the reference; the Triton launches are replaced by ``mta_headmix_fwd``,
``mta_headmix_bwd_input`` and ``mta_headmix_bwd_weight``.  One addition: an optional
``group_size`` hint.  The reference weight is always a dense (H,H) matrix; when it is
block diagonal, passing the block size lets the kernels skip the zero blocks (the result
is identical); the weight gradient is then confined to the blocks as well, so that an
optimizer step keeps the structure the caller promised.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from . import ops


class TritonLinearHeadFunction(torch.autograd.Function):
    """apply(input (N,C,P,Q), weight (C,C), causal=True, output_value=0.0[, group_size]).

    Two optional flags for callers that know who reads the results (both only matter when ``causal``):
    ``fill_upper=False`` -- the output is only read on and below the diagonal; ``grad_fill_upper=False`` -- so is the
    input gradient that backward returns.  What lies above the diagonal is then left unwritten."""

    @staticmethod
    def forward(ctx, input, weight, causal=True, output_value=0.0, group_size=None, fill_upper=True,
                grad_fill_upper=True):
        ctx.save_for_backward(input, weight)
        ctx.causal = causal
        ctx.group_size = group_size
        ctx.grad_fill_upper = grad_fill_upper
        return ops.headmix(input, weight, causal, output_value, group_size, fill_upper=fill_upper)

    @staticmethod
    def backward(ctx, grad_output):
        """triton_linear_head.py:322-370.  Above the diagonal the input gradient is 0 (the reference leaves
        ``torch.empty_like`` memory there); the weight gradient is accumulated in fp32 and cast."""
        input, weight = ctx.saved_tensors
        grad_input = grad_weight = None
        if ctx.needs_input_grad[0]:
            grad_input = ops.headmix_bwd_input(grad_output, weight, ctx.causal, ctx.group_size,
                                               fill_upper=ctx.grad_fill_upper)
        if ctx.needs_input_grad[1]:
            grad_weight = ops.headmix_bwd_weight(input, grad_output.to(input.dtype), ctx.causal)
            if ctx.group_size:
                blk = torch.arange(weight.shape[0], device=weight.device) // ctx.group_size
                grad_weight = grad_weight * (blk[:, None] == blk[None, :])
            grad_weight = grad_weight.to(weight.dtype)
        return grad_input, grad_weight, None, None, None, None, None


class TritonLinearHead(nn.Module):
    """y[b,o,p,q] = sum_i weight[o,i] x[b,i,p,q]; above the diagonal holds ``output_value`` when causal."""

    def __init__(self, head_dim, causal=True, output_value=0.0, group_size=None):
        super().__init__()
        self.head_dim = head_dim
        self.causal = causal
        self.output_value = output_value
        self.group_size = group_size
        # same default draw as triton_linear_head.py:384
        self.weight = nn.Parameter(torch.randn(head_dim, head_dim) / (head_dim ** 0.5))

    def forward(self, x):
        return TritonLinearHeadFunction.apply(x, self.weight, self.causal, self.output_value, self.group_size)

    def extra_repr(self):
        return f"head_dim={self.head_dim}"
