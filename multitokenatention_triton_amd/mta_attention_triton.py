"""Multi-Token Attention module (HIP-backed), drop-in for the reference's MTAAttentionTriton.

Same constructor, attribute names, parameter names and forward signature as
mta_attention_triton.py:7-201, so state dicts and calling code carry over.  What differs
is how forward() is executed on the GPU (the values are those of
mta_attention_pytorch.py:58-83):

  * the 1/sqrt(D) factor is applied by the pre-softmax conv while it stages its tile
    (``mta_conv2d_scaled_fwd``) instead of a separate pass over the (B,H,S,S) scores;
  * pre-softmax head mixing, the causal mask, the fp32 softmax and -- when the
    post-softmax conv kernel is the identity tap -- the post-softmax head mixing run
    as one kernel (``mta_headmix_softmax_fwd``): one pass over the score tensor
    instead of four, and no fp32 copy of it;
  * block-diagonal head-mixing weights are detected and only their blocks are applied.

Weight structure (identity conv tap, identity / block-diagonal head weights) is probed on
the host and remembered per parameter, keyed by the parameter's autograd version counter
and storage address.  Optimizer steps, ``load_state_dict``, ``copy_`` under ``no_grad`` and
this module's own reset/copy methods all move that counter.  A write through ``.data``
does not: after one, call ``refresh_structure()`` (or construct the module with
``weight_structure="dense"``, which never assumes any structure).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops
from .convolution_2d_trit import Conv2dTriton
from .triton_linear_head import TritonLinearHead

# largest mixing group the one-pass mix/softmax/mix kernel keeps in registers
_FUSED_MAX_GROUP = 8


@dataclass
class MTAConfig:
    """The attribute bag the reference passes as ``mta`` (compare_mta_attention.py:7-18)."""
    use_mta: bool = True
    query_kernel_size: int = 3
    key_kernel_size: int = 3
    after_sm_query_kernel_size: int = 3
    after_sm_key_kernel_size: int = 3
    pre_sm_linear_head: bool = True
    post_sm_linear_head: bool = True
    pad_key: str = "both"
    init_method: str = "identity"
    dim: int = 512


class MTAAttentionTriton(nn.Module):
    def __init__(self, n_heads: int, mta, dropout: float, causal: bool, use_mask: bool = False):
        super().__init__()
        assert mta.use_mta, "MTAAttentionTriton can only be used with MTA"
        assert mta.query_kernel_size is not None and mta.key_kernel_size is not None
        assert mta.pre_sm_linear_head is True
        for name, default in (("after_sm_query_kernel_size", 3), ("after_sm_key_kernel_size", 3),
                              ("post_sm_linear_head", True)):
            if not hasattr(mta, name):
                setattr(mta, name, default)

        self.n_heads = n_heads
        self.mta = mta
        self.dropout = dropout
        self.causal = causal
        self.use_mask = use_mask
        self.pad_key = mta.pad_key
        self.mta_init_method = mta.init_method

        self.mta_conv_triton = Conv2dTriton(n_heads, (mta.query_kernel_size, mta.key_kernel_size), causal=causal)
        self.wpsm_triton = TritonLinearHead(n_heads, causal=causal, output_value=float("-inf"))
        self.mta_conv_after_sm_triton = Conv2dTriton(
            n_heads, (mta.after_sm_query_kernel_size, mta.after_sm_key_kernel_size), causal=causal)
        self.wposm_triton = TritonLinearHead(n_heads, causal=causal)
        # optional observer: called as hook(stage_name) right before each stage is enqueued
        self._stage_hook = None
        # "auto": probe weight structure and pick specialised kernels; "dense": assume nothing
        self.weight_structure = "auto"
        self._structure = {}

    # ------------------------------------------------------------------ forward
    def _mark(self, name: str) -> None:
        if self._stage_hook is not None:
            self._stage_hook(name)

    def forward(self, xq, xk, xv, mask, chunk_start_ids):
        assert chunk_start_ids is None, "MTAAttentionTriton does not support chunked attention"
        if self.use_mask:
            return self._forward_with_mask(xq, xk, xv, mask)

        head_dim = xq.size(-1)
        # the reference multiplies by rsqrt(tensor(head_dim)), an fp32 scalar (mta_attention_triton.py:69-71)
        scale = float(torch.rsqrt(torch.tensor(float(head_dim))))
        w_pre, w_post = self.wpsm_triton.weight, self.wposm_triton.weight
        pre_eye, g_pre = self._probe("wpsm", w_pre, _probe_head)
        post_eye, g_post = self._probe("wposm", w_post, _probe_head)
        post_conv_identity = self._probe("conv_post", self.mta_conv_after_sm_triton.weight, _probe_conv)
        w1 = None if pre_eye else w_pre
        w2 = None if post_eye else w_post
        one_pass = post_conv_identity and _lcm(g_pre, g_post) <= _FUSED_MAX_GROUP
        # the last stage may leave the upper triangle unwritten only if our own P V kernel consumes it
        own_pv = (xq.size(-2) == xk.size(-2) and xq.dtype == xv.dtype
                  and ops.causal_pv_supported(xq.dtype, xq.size(-2), xv.size(-1)))

        # QK^T -> *1/sqrt(d) -> conv: one kernel when it exists for this dtype / size, else GEMM + conv
        self._mark("qk_conv")
        scores = None
        if xq.shape == xk.shape:
            scores = ops.qk_conv(xq, xk, self.mta_conv_triton.weight, self.causal, scale, fill_upper=False)
        if scores is None:
            self._mark("qk")
            scores = torch.matmul(xq, xk.transpose(2, 3))
            self._mark("conv_pre")
            scores = ops.conv2d_causal(scores, self.mta_conv_triton.weight, self.causal, in_scale=scale)

        if one_pass:
            self._mark("mix_softmax_mix")
            scores = ops.headmix_softmax(scores, w1, w2, self.causal, group_size=_lcm(g_pre, g_post),
                                         fill_upper=not own_pv)
        else:
            if g_pre <= _FUSED_MAX_GROUP:
                self._mark("mix_softmax")
                scores = ops.headmix_softmax(scores, w1, None, self.causal, group_size=g_pre,
                                             fill_upper=post_conv_identity and w2 is None and not own_pv)
            else:
                self._mark("mix_pre")
                fill = float("-inf") if self.causal else 0.0
                scores = ops.headmix(scores, w_pre, self.causal, fill, group_size=g_pre)
                self._mark("softmax")
                scores = ops.headmix_softmax(scores, None, None, self.causal,
                                             fill_upper=post_conv_identity and w2 is None and not own_pv)
            if not post_conv_identity:
                self._mark("conv_post")
                scores = ops.conv2d_causal(scores, self.mta_conv_after_sm_triton.weight, self.causal)
            if w2 is not None:
                self._mark("mix_post")
                scores = ops.headmix(scores, w_post, self.causal, 0.0, group_size=g_post)

        scores = F.dropout(scores, p=self.dropout, training=self.training)
        self._mark("pv")
        output = ops.causal_pv(scores, xv, self.causal) if own_pv else None
        if output is None:
            output = torch.matmul(scores, xv)
        self._mark("end")
        return output.transpose(1, 2)

    def _probe(self, name, weight, fn):
        if self.weight_structure != "auto":
            return (False, self.n_heads) if fn is _probe_head else False
        key = (id(weight), weight._version, weight.data_ptr(), weight.dtype)
        hit = self._structure.get(name)
        if hit is None or hit[0] != key:
            hit = (key, fn(weight))
            self._structure[name] = hit
        return hit[1]

    def refresh_structure(self):
        """Forget what was learnt about the weights' structure (needed after writes through ``.data``)."""
        self._structure.clear()

    def _forward_with_mask(self, xq, xk, xv, mask):
        """use_mask=True: an explicit additive mask tensor drives the masking (mta_attention_triton.py:63-64,
        77-83, 96-98); the kernels still apply their own causal rule when ``causal`` is set."""
        mask = self._update_mask(mask=mask, bsz=xq.size(0), xq=xq, xk_size=xk.size(-2))
        scale = torch.rsqrt(torch.tensor(float(xq.size(-1)), device=xq.device))
        scores = torch.matmul(xq, xk.transpose(2, 3)) * scale
        blocked = mask == float("-inf")
        scores = self.mta_conv_triton(scores.masked_fill(blocked, 0))
        scores = self.wpsm_triton(scores)
        scores = scores + mask
        scores = F.softmax(scores.float(), dim=-1).type_as(xq)
        scores = self.mta_conv_after_sm_triton(scores.masked_fill(blocked, 0))
        scores = torch.where(blocked, 0.0, scores)
        scores = self.wposm_triton(scores)
        scores = F.dropout(scores, p=self.dropout, training=self.training)
        return torch.matmul(scores, xv).transpose(1, 2)

    def _update_mask(self, mask, bsz: int, xq: torch.Tensor, xk_size: int):
        """Additive (B,H,Sq,Sk) mask, 0 = attend, -inf = blocked (mta_attention_triton.py:106-127)."""
        sq = xq.size(-2)
        if not isinstance(mask, torch.Tensor):
            mask = torch.triu(torch.full((sq, xk_size), float("-inf"), device=xq.device), diagonal=1).type_as(xq)
            return mask.repeat(bsz, self.n_heads, 1, 1)
        if mask.dtype == torch.bool:
            mask = torch.where(mask, 0.0, float("-inf")).to(xq.dtype)
        if mask.dtype != xq.dtype:
            mask = mask.type(xq.dtype)
        if mask.dim() == 2:
            assert mask.size(0) == bsz
            mask = mask.repeat(1, self.n_heads, sq, 1)
            rows, cols = torch.triu_indices(sq, xk_size, offset=1)
            mask[:, :, rows, cols] = float("-inf")
        elif mask.size(0) == 1 and mask.size(1) == 1:
            mask = mask.repeat(bsz, self.n_heads, 1, 1)
        return mask

    # ------------------------------------------------------------------ parameters
    def reset_mta_parameters(self, init_std=None):
        """Conv kernels per ``mta.init_method``; both head-mixing weights to the identity
        (mta_attention_triton.py:129-146)."""
        init_std = init_std or (self.mta.dim ** (-0.5))
        self._init_conv_kernel(self.mta_conv_triton.weight, init_std)
        self._init_conv_kernel(self.mta_conv_after_sm_triton.weight, init_std)
        with torch.no_grad():
            nn.init.eye_(self.wpsm_triton.weight)
            nn.init.eye_(self.wposm_triton.weight)

    def _init_conv_kernel(self, kernel, init_std):
        method = self.mta_init_method
        with torch.no_grad():
            if method == "uniform":
                kernel.uniform_(-1.0, 1.0)
            elif method == "normal":
                # the reference calls uniform_ with normal-style arguments here and raises
                # (mta_attention_triton.py:152-160); a truncated normal is what those arguments describe
                nn.init.trunc_normal_(kernel, mean=0.0, std=0.3, a=-0.9, b=0.9)
            elif method == "diagonal":
                _, rows, cols = kernel.shape
                offset = (cols + 1) // 2 - rows
                band = torch.ones(rows, cols, dtype=kernel.dtype, device=kernel.device)
                kernel.copy_(torch.triu(torch.tril(band, offset), offset).expand_as(kernel))
            elif method == "identity":
                assert self.pad_key == "both"
                kernel.zero_()
                kernel[:, -1, kernel.shape[-1] // 2] = 1.0
            elif method == "const":
                kernel.fill_(0.3)
            else:
                raise ValueError(f"Unsupported mta_init_method: {method}")

    def copy_mta_parameters(self, mta_attention):
        """Take the four weights of a PyTorch MTAAttention; its conv kernels are (H,1,R,S)
        (mta_attention_triton.py:185-201)."""
        with torch.no_grad():
            if hasattr(mta_attention, "mta_kernel"):
                self.mta_conv_triton.weight.copy_(mta_attention.mta_kernel.data.squeeze(1))
            if hasattr(mta_attention, "mta_kernel_after_sm"):
                self.mta_conv_after_sm_triton.weight.copy_(mta_attention.mta_kernel_after_sm.data.squeeze(1))
            if hasattr(mta_attention, "wpsm"):
                self.wpsm_triton.weight.copy_(mta_attention.wpsm.weight.data)
            if hasattr(mta_attention, "wposm"):
                self.wposm_triton.weight.copy_(mta_attention.wposm.weight.data)


def _probe_head(w):
    """(is identity, block-diagonal group size)."""
    if ops.is_identity_head_weight(w):
        return True, 1
    return False, ops.block_diagonal_group(w)


def _probe_conv(w):
    return ops.is_identity_conv_kernel(w)


def _lcm(a: int, b: int) -> int:
    import math
    return a * b // math.gcd(a, b)


__all__ = ["MTAAttentionTriton", "MTAConfig"]
_ = Optional
