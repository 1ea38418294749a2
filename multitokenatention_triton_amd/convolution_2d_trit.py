"""Depthwise causal 2-D convolution operator (HIP-backed).

Mirrors the public names of the reference's convolution_2d_trit.py -- Conv2dTriton
(:381-401) and Conv2dTritonFunction (:300-333) -- so modules written against it keep
working; the Triton launch is replaced by ``mta_conv2d_fwd`` of libmta_hip.so.
Forward only: the reference's backward kernels (:143-295) are outside this build.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from . import ops


class Conv2dTritonFunction(torch.autograd.Function):
    """apply(input (N,C,H,W), weight (C,R,S), causal) -> (N,C,H,W), same dtype as input."""

    @staticmethod
    def forward(ctx, input, weight, causal):
        return ops.conv2d_causal(input, weight, causal)

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("the HIP build of Conv2dTritonFunction is forward-only")


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
