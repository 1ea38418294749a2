"""Head-axis linear ("head mixing") operator (HIP-backed).

Mirrors TritonLinearHead (triton_linear_head.py:373-401) and TritonLinearHeadFunction
(:281-319) of the reference; the Triton launch is replaced by ``mta_headmix_fwd``.
Forward only.  One addition: an optional ``group_size`` hint.  The reference weight is
always a dense (H,H) matrix; when it is block diagonal, passing the block size lets the
kernel skip the zero blocks (the result is identical).
"""
from __future__ import annotations

import torch
import torch.nn as nn

from . import ops


class TritonLinearHeadFunction(torch.autograd.Function):
    """apply(input (N,C,P,Q), weight (C,C), causal=True, output_value=0.0[, group_size])."""

    @staticmethod
    def forward(ctx, input, weight, causal=True, output_value=0.0, group_size=None):
        return ops.headmix(input, weight, causal, output_value, group_size)

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("the HIP build of TritonLinearHeadFunction is forward-only")


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
