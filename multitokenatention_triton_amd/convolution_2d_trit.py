"""Depthwise causal 2-D convolution operator (HIP-backed).

Mirrors the public names of the reference's convolution_2d_trit.py -- Conv2dTriton
(:381-401), Conv2dTritonFunction (:300-378), PytorchConv / pytorch_conv /
add_causal_mask (:404-432) -- so modules written against it keep working.  The Triton
launches are replaced by ``mta_conv2d_fwd``, ``mta_conv2d_bwd_input`` and
``mta_conv2d_bwd_weight`` of libmta_hip.so.
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops


class Conv2dTritonFunction(torch.autograd.Function):
    """apply(input (N,C,H,W), weight (C,R,S), causal) -> (N,C,H,W), same dtype as input.

    Two optional flags for callers that know who reads the results (both only matter when ``causal``):
    ``fill_upper=False`` -- the output is only read on and below the diagonal; ``grad_fill_upper=False`` -- so is the
    input gradient that backward returns.  What lies above the diagonal is then left unwritten."""

    @staticmethod
    def forward(ctx, input, weight, causal, fill_upper=True, grad_fill_upper=True):
        ctx.save_for_backward(input, weight)
        ctx.causal = causal
        ctx.grad_fill_upper = grad_fill_upper
        return ops.conv2d_causal(input, weight, causal, fill_upper=fill_upper)

    @staticmethod
    def backward(ctx, grad_output):
        """convolution_2d_trit.py:336-378.  The reference returns the weight gradient in fp64 and lets autograd
        cast it; here it is accumulated in fp32 and cast to the weight's dtype."""
        input, weight = ctx.saved_tensors
        grad_input = grad_weight = None
        if ctx.needs_input_grad[0]:
            grad_input = ops.conv2d_bwd_input(grad_output, weight, ctx.causal, fill_upper=ctx.grad_fill_upper)
        if ctx.needs_input_grad[1]:
            grad_weight = ops.conv2d_bwd_weight(input, grad_output.to(input.dtype), tuple(weight.shape[1:]),
                                                ctx.causal).to(weight.dtype)
        return grad_input, grad_weight, None, None, None


class Conv2dTriton(nn.Module):
    """Holds the (channels, R, S) kernel; ``kernel_size`` is an int or an (R,S) tuple."""

    def __init__(self, channels, kernel_size, causal=False):
        super().__init__()
        self.channels = channels
        self.kernel_size = tuple(kernel_size) if isinstance(kernel_size, (tuple, list)) else (kernel_size, kernel_size)
        self.causal = causal
        self.weight = nn.Parameter(torch.empty(channels, *self.kernel_size))
        self._init_parameters()

    def _init_parameters(self):
        # Default of the reference (convolution_2d_trit.py:393-398): a single 1.0 at the
        # geometric centre [R//2, S//2].  With top-only row padding this is a pass-through
        # only when R == 1; MTA modules overwrite it through reset_mta_parameters().
        with torch.no_grad():
            self.weight.zero_()
            self.weight[:, self.kernel_size[0] // 2, self.kernel_size[1] // 2] = 1.0

    def forward(self, x):
        return Conv2dTritonFunction.apply(x, self.weight, self.causal)

    def extra_repr(self):
        return f"channels={self.channels}, kernel_size={self.kernel_size}, causal={self.causal}"


def add_causal_mask(x):
    """x with everything above the diagonal zeroed (convolution_2d_trit.py:404-406)."""
    return x * torch.tril(torch.ones_like(x))


def pytorch_conv(x, weight, causal=False):
    """The reference's library restatement of the operator (convolution_2d_trit.py:418-432): pad R-1 rows on top and
    (S-1)//2 keys on both sides, grouped F.conv2d with a (C,1,R,S) weight, output masked when causal.  Unlike the
    kernels it does not mask its *input*; it runs wherever its tensors live and is not backed by libmta_hip."""
    qdim, kdim = weight.shape[-2], weight.shape[-1]
    padded = F.pad(x, ((kdim - 1) // 2, (kdim - 1) // 2, qdim - 1, 0), value=0.0)
    out = F.conv2d(padded, weight, padding=0, groups=x.shape[1])
    return add_causal_mask(out) if causal else out


class PytorchConv(nn.Module):
    """Parameter holder around ``pytorch_conv`` (convolution_2d_trit.py:408-416); weight is (C,1,R,S)."""

    def __init__(self, channels, kernel_size, causal=False):
        super().__init__()
        self.kernel_size = tuple(kernel_size) if isinstance(kernel_size, (tuple, list)) else (kernel_size, kernel_size)
        self.weight = nn.Parameter(torch.randn(channels, 1, self.kernel_size[0], self.kernel_size[1]))
        self.causal = causal

    def forward(self, x):
        return pytorch_conv(x, self.weight, self.causal)
