"""Multi-Token Attention module (HIP-backed), drop-in for the reference's MTAAttentionTriton.

Same constructor, attribute names, parameter names and forward signature as
mta_attention_triton.py:7-201, so state dicts and calling code carry over.  What differs
is how forward() is executed on the GPU (the values are those of
mta_attention_pytorch.py:58-83).

Inference (no input or parameter requires grad, or grad mode is off):

  * QK^T, the 1/sqrt(D) factor and the pre-softmax conv run as one kernel
    (``mta_qk_conv_fwd``): the raw scores never reach HBM;
  * pre-softmax head mixing, the causal mask, the fp32 softmax and -- when the
    post-softmax conv kernel is the identity tap -- the post-softmax head mixing run
    as one kernel (``mta_headmix_softmax_fwd``): one pass over the score tensor
    instead of four, and no fp32 copy of it;
  * otherwise, for mixing groups of up to 4 heads and 3x3 or 7x7 kernels, and for dense
    groups of 16 heads and 3x3, 5x5 or 7x7 kernels, the post-softmax conv and head mixing
    run as one kernel (``mta_conv2d_headmix_fwd``): the conv result never reaches HBM;
  * P V reads only the lower triangle of P (``mta_causal_pv_fwd``);
  * where all of these kernels know it, the score tensors between them travel in a
    triangular layout (``mta_qk_conv_tri_fwd`` and its two companions): the lower triangle
    only, the rows one kernel reads side by side (``score_layout = "planes"`` keeps
    (B,H,S,S) tensors);
  * ``use_mask=True``: masks that amount to "the causal rule and hidden keys" (2-D key
    masks, key padding of a batch) or to "row p sees the keys first[p] .. p" (sliding
    windows, packed documents) go into the same kernels as one value per key or per row
    (a ``causal=False`` module: masks that hide the same keys from every row, the key
    padding of an encoder batch); any other boolean or additive mask (holes, a plane per
    head, finite values) runs on the single-stage kernels with the reference's three
    elementwise mask steps as passes over a byte per position (``mta_mask_fill_fwd``;
    ``mta_mask_add_fwd`` for finite values); only lengths that are not a multiple of 8 take
    the reference's elementwise steps around the kernels.

Training (something requires grad): the stages run one by one through autograd
Functions, as in the reference, so that ``backward()`` works: the two conv and the two
head-mixing stages with their HIP gradient kernels (convolution_2d_trit /
triton_linear_head); the 1/sqrt(D) factor folded into the pre-softmax conv and, in
backward, into the (B,H,S,D) gradients of Q and K; pre-softmax head mixing and softmax as
one forward kernel where the inference route has one, with the softmax gradient taken from
the stored 16-bit probabilities (``mta_softmax_bwd``; no fp32 copy of the score tensor in
either direction).  Under the causal rule the products around the score tensors (P V, the
gradients it leaves, the recomputed raw scores) touch the lower triangle only; torch
differentiates the dropout.  ``use_mask=True`` in training: the same two families of masks
go through these operators -- hidden keys as a key bias inside the softmax kernel and
zeroed K and V rows, band masks inside the scores and softmax kernels, with the gradients
around them formed inside the band; masks of arbitrary content as mask passes between the
operators, whose gradients they zero at the same positions.

Weight structure.  By default nothing is assumed about the four weights: every stage runs
with the dense weight it is given.  Skipping identity stages and applying block-diagonal
head weights block by block is an explicit opt-in, because a parameter can be rewritten
behind the module's back (``p.data.copy_(...)`` leaves no trace on the host):

  * ``infer_weight_structure()`` looks at the current weights once (on the device, one
    small read back) and keeps what it found until told otherwise;
  * ``declare_weight_structure(...)`` states it without looking;
  * ``weight_structure = "probe"`` looks on every call (one tiny launch and a
    synchronising 20-byte read per forward; not usable under stream capture);
  * ``assume_dense_weights()`` returns to the default.

``reset_mta_parameters``, ``copy_mta_parameters`` and ``load_state_dict`` return to the
default as well.  A declared structure is the caller's promise, like ``group_size`` in the
C ABI: weights that break it give results for the declared structure.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import os

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops
from .convolution_2d_trit import Conv2dTriton, Conv2dTritonFunction
from .triton_linear_head import TritonLinearHead, TritonLinearHeadFunction

# largest mixing group the one-pass mix/softmax/mix kernel keeps in registers ...
_FUSED_MAX_GROUP = 8
# ... and the group size its matrix-core variant takes (16-bit data, rows of up to _FUSED_MFMA_MAX_KEYS keys)
_FUSED_MFMA_GROUP = 16
_FUSED_MFMA_MAX_KEYS = 4096


def _one_pass_group(group: int, scores_dtype, n_keys: int, *weights) -> bool:
    """Whether mix -> softmax (-> mix) over mixing groups of ``group`` heads runs as one kernel."""
    if group <= _FUSED_MAX_GROUP:
        return True
    return (group == _FUSED_MFMA_GROUP and scores_dtype in (torch.bfloat16, torch.float16)
            and n_keys % 8 == 0 and n_keys <= _FUSED_MFMA_MAX_KEYS
            and all(w is None or w.dtype == scores_dtype for w in weights))
# where the one-pass post-softmax conv + head mixing kernel is used (see forward)
_CONV_MIX_MAX_GROUP = 4
_CONV_MIX_SIZES = ((3, 3), (7, 7))
# ... and for dense groups of 16 heads at 16-bit dtypes (conv and mixing both on the matrix cores)
_CONV_MIX16_SIZES = ((3, 3), (5, 5), (7, 7))


_IDENTITY_KERNELS = {}


def _lower_scores(a: torch.Tensor, b: torch.Tensor, first_visible: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """round(a b^T) on and below the diagonal of a (B,H,S,S) tensor, nothing written above it, for consumers that
    never read there: the scores kernel (``mta_qk_conv_fwd``) with factor 1 and a 3x3 kernel that is the pass-through
    tap, which copies its input exactly.  Half the output traffic of the library GEMM.  None where that kernel does not
    apply (fp32, ragged lengths): the caller then takes the GEMM."""
    if a.shape != b.shape or a.dtype == torch.float32 or a.dtype != b.dtype:
        return None
    h = a.size(1)
    key = (h, a.dtype, a.device)
    w = _IDENTITY_KERNELS.get(key)
    if w is None:
        w = torch.zeros(h, 3, 3, dtype=a.dtype, device=a.device)
        w[:, 2, 1] = 1.0
        _IDENTITY_KERNELS[key] = w
    out = ops.qk_conv(a, b, w, True, 1.0, fill_upper=False, first_visible=first_visible)
    if out is not None and first_visible is not None:
        # a band mask: the products ahead of a row's first visible key count as 0.  The kernel does not visit the key
        # blocks that no row of a query block sees: the hidden stretch of every row is cleared afterwards.
        out = ops.band_zero_(out, first_visible)
    return out


class _ProbsTimesValues(torch.autograd.Function):
    """P V of the training route (mta_attention_triton.py:89).  When ``lower`` (causal: the producer of P wrote nothing
    above the diagonal, and the head mixing's gradient kernels, which take dP from here, read nothing there) all three
    products touch the lower triangle of their (B,H,S,S) operand only: forward ``mta_causal_pv_fwd``, dV = P^T dO
    ``mta_causal_ptx_fwd``, dP = dO V^T ``_lower_scores``.  Where those kernels do not apply (fp32, ragged lengths, other
    head sizes) the caller has filled P and the library GEMMs run."""

    @staticmethod
    def forward(ctx, p, v, lower, first_visible=None):
        # (first_visible: a band mask, P is 0 ahead of every row's first visible key; needs ``lower``.  The gradient with
        # respect to P is then formed inside the band only: 0 at the hidden positions, where the reference's
        # ``torch.where(mask == -inf, 0.0, scores)`` cuts it)
        assert first_visible is None or lower
        ctx.save_for_backward(p, v, first_visible)
        ctx.lower = lower
        out = ops.causal_pv(p, v, True, first_visible=first_visible) if lower else None
        return out if out is not None else torch.matmul(p, v)

    @staticmethod
    def backward(ctx, grad_output):
        p, v, first_visible = ctx.saved_tensors
        dp = dv = None
        if ctx.needs_input_grad[0]:
            dp = _lower_scores(grad_output, v, first_visible) if ctx.lower else None
            if dp is None:
                assert first_visible is None
                dp = torch.matmul(grad_output, v.transpose(2, 3))
        if ctx.needs_input_grad[1]:
            dv = ops.causal_ptx(p, grad_output.contiguous(), True) if ctx.lower else None
            if dv is None:
                dv = torch.matmul(p.transpose(2, 3), grad_output)
        return dp, dv, None, None


def _lower_products_supported(x: torch.Tensor, s_keys: int) -> bool:
    """Whether P V, P^T X and round(a b^T) run as kernels that read / write the lower triangle only."""
    return x.size(-2) == s_keys and ops.causal_pv_supported(x.dtype, s_keys, x.size(-1))


class _ScaledScoresConv(torch.autograd.Function):
    """conv(round(Q K^T) * scale) for the training route (mta_attention_triton.py:69-73).  Forward: the inference
    route's one kernel (``mta_qk_conv_fwd``, the raw scores never reach memory) where it exists; otherwise the library
    GEMM, then ``mta_conv2d_scaled_fwd``, which applies the factor (and the rounding to the score dtype that the
    reference's separate multiplication performs) on the way into the conv.  Backward: the conv's input gradient ``g``
    goes through the two products dQ = G K and dK = G^T Q and the factor is applied to their (B,H,S,D) results - under
    the causal rule with ``mta_causal_pv_fwd`` and ``mta_causal_ptx_fwd``, which read the lower triangle of ``g`` only (it
    is then not written above the diagonal either), else with the library GEMMs; the kernel gradient is taken against
    the raw scores -- kept by the second forward, recomputed with one product after the first, which so saves a
    (B,H,S,S) activation -- and scaled afterwards.  Neither direction spends a pass over a (B,H,S,S) tensor on the
    factor."""

    @staticmethod
    def forward(ctx, xq, xk, weight, scale, causal, mark, first_visible=None, mask_planes=None):
        # (first_visible: a band mask, applied to the scores ahead of the conv (mta_attention_triton.py:72-73) inside the
        # one kernel, which the caller has checked exists; backward: the conv's input gradient is zeroed at the hidden
        # positions, the raw scores for the kernel gradient are recomputed inside the band)
        # (mask_planes: uint8 (1|B, 1|H, S, S), a mask of arbitrary content: the raw scores are written, the hidden ones
        # zeroed in place, and kept for the kernel gradient; backward zeroes the conv's input gradient at the same positions)
        ctx.scale, ctx.causal, ctx.first_visible, ctx.mask_planes = scale, causal, first_visible, mask_planes
        if mask_planes is not None:
            assert first_visible is None
            mark("qk")
            raw = _lower_scores(xq, xk) if causal else None
            if raw is None:
                raw = torch.matmul(xq, xk.transpose(2, 3))
            mark("mask")
            if ops.mask_fill(raw, mask_planes, False, causal, out=raw) is None:
                raise RuntimeError("mask planes need a number of keys that is a multiple of 8")
            mark("conv_pre")
            ctx.save_for_backward(xq, xk, weight, raw)
            return ops.conv2d_causal(raw, weight, causal, in_scale=scale, fill_upper=False)
        # (the stage that follows, head mixing or mixing + softmax, never reads above the diagonal)
        if ops.qk_conv_supported(xq, xk, weight):
            mark("qk_conv")
            out = ops.qk_conv(xq, xk, weight, causal, scale, fill_upper=False, first_visible=first_visible)
            if out is not None and first_visible is not None:
                # The kernel leaves the key blocks that no row of a query block sees unwritten.  The softmax stage does not
                # read a row's hidden stretch, but its weight gradient multiplies what is stored there by a gradient that
                # is 0: the stretch is cleared, so that the product is 0 too.
                out = ops.band_zero_(out, first_visible)
            if out is not None:
                ctx.save_for_backward(xq, xk, weight, None)
                return out
        assert first_visible is None, "the band mask needs the one-kernel first stage"
        mark("qk")
        raw = torch.matmul(xq, xk.transpose(2, 3))
        mark("conv_pre")
        ctx.save_for_backward(xq, xk, weight, raw)
        return ops.conv2d_causal(raw, weight, causal, in_scale=scale, fill_upper=False)

    @staticmethod
    def backward(ctx, grad_output):
        xq, xk, weight, raw = ctx.saved_tensors
        dq = dk = dw = None
        if ctx.needs_input_grad[0] or ctx.needs_input_grad[1]:
            lower = ctx.causal and xq.shape == xk.shape and _lower_products_supported(xq, xk.size(-2))
            g = ops.conv2d_bwd_input(grad_output, weight, ctx.causal, fill_upper=not lower)
            if ctx.first_visible is not None:
                assert lower
                if ops.band_zero_(g, ctx.first_visible) is None:
                    raise RuntimeError("band masks need 16-bit scores of a length that is a multiple of 8")
            if ctx.mask_planes is not None:
                ops.mask_fill(g, ctx.mask_planes, False, lower, out=g)
            if ctx.needs_input_grad[0]:
                dq = ops.causal_pv(g, xk, True) if lower else None
                if dq is None:
                    assert not lower
                    dq = torch.matmul(g, xk)
                dq = dq * ctx.scale
            if ctx.needs_input_grad[1]:
                dk = ops.causal_ptx(g, xq, True) if lower else None
                if dk is None:
                    assert not lower
                    dk = torch.matmul(g.transpose(2, 3), xq)
                dk = dk * ctx.scale
        if ctx.needs_input_grad[2]:
            if raw is None:  # (the kernel gradient reads its first argument on and below the diagonal only)
                raw = _lower_scores(xq, xk, ctx.first_visible) if ctx.causal else None
                if raw is None:
                    assert ctx.first_visible is None
                    raw = torch.matmul(xq, xk.transpose(2, 3))
            dw = ops.conv2d_bwd_weight(raw, grad_output.to(raw.dtype), tuple(weight.shape[1:]), ctx.causal)
            dw = (dw * ctx.scale).to(weight.dtype)
        return dq, dk, dw, None, None, None, None, None


class _MaskFill(torch.autograd.Function):
    """``visible ? x : fill`` in place for uint8 visibility planes (``mta_mask_fill_fwd``).  fill = -inf is the
    reference's ``scores + mask`` ahead of the softmax (mta_attention_triton.py:77-78): the gradient is handed on as it
    is, because the softmax that follows returns exactly 0 where its probabilities are 0.  fill = 0 is its
    ``torch.where(mask == -inf, 0.0, scores)`` behind the post-softmax conv (:82-83): the gradient is zeroed at the same
    positions, into a tensor of its own."""

    @staticmethod
    def forward(ctx, x, planes, neg_inf, causal):
        if ops.mask_fill(x, planes, neg_inf, causal, out=x) is None:
            raise RuntimeError("mask planes need a number of keys that is a multiple of 8")
        ctx.mark_dirty(x)
        ctx.neg_inf, ctx.causal = neg_inf, causal
        ctx.save_for_backward(planes)
        return x

    @staticmethod
    def backward(ctx, grad_output):
        if ctx.neg_inf:
            return grad_output, None, None, None
        planes, = ctx.saved_tensors
        return ops.mask_fill(grad_output.contiguous(), planes, False, ctx.causal), None, None, None


class _MaskAdd(torch.autograd.Function):
    """``x + mask`` in place (``mta_mask_add_fwd``): the reference's ``scores + mask`` ahead of the softmax for an additive
    mask with finite values.  The gradient is handed on as it is: the derivative is 1, and where the mask is -inf the
    softmax that follows returns exactly 0."""

    @staticmethod
    def forward(ctx, x, mask, causal):
        if ops.mask_add(x, mask, causal, out=x) is None:
            raise RuntimeError("mask planes need a number of keys that is a multiple of 8")
        ctx.mark_dirty(x)
        return x

    @staticmethod
    def backward(ctx, grad_output):
        return grad_output, None, None


class _BandZero(torch.autograd.Function):
    """x[b,h,p,q] = 0 for q < first_visible[b,p], in place: what ``torch.where(mask == -inf, 0.0, scores)`` behind the
    post-softmax conv does under a band mask (mta_attention_triton.py:82-83).  Its gradient would be the same zeroing;
    here the gradient that arrives is zero at those positions already - the gradient with respect to the probabilities
    is formed inside the band only (``_ProbsTimesValues``) and what lies between, dropout and head mixing, acts per
    position - so it is handed on as it is."""

    @staticmethod
    def forward(ctx, x, first_visible):
        if ops.band_zero_(x, first_visible) is None:
            raise RuntimeError("band masks need 16-bit scores of a length that is a multiple of 8")
        ctx.mark_dirty(x)
        return x

    @staticmethod
    def backward(ctx, grad_output):
        return grad_output, None


class _MixSoftmax(torch.autograd.Function):
    """softmax(mix(x, weight)) over the keys for the training route (mta_attention_triton.py:75-79), one kernel
    (``mta_headmix_softmax_fwd``; ``weight=None``: the softmax alone).  The probabilities are computed in fp32 from the
    mixed scores rounded to the score dtype and stored in it, as ``F.softmax(scores.float()).type_as(scores)`` leaves
    them.  Backward: the softmax gradient from the stored probabilities (``mta_softmax_bwd``), then the head mixing's
    two gradient kernels."""

    @staticmethod
    def forward(ctx, x, weight, causal, group_size, fill_upper=True, grad_fill_upper=True, key_bias=None,
                first_visible=None, zero_planes=None):
        # (key_bias: fp32 (B,Sk) added to the mixed scores, 0 or -inf per key; first_visible: int32 (B,S), a band mask.
        # Constants: the gradient is the softmax's own, taken from the stored probabilities, which are 0 at what is hidden)
        p = ops.headmix_softmax(x, weight, None, causal, group_size=group_size if weight is not None else None,
                                fill_upper=fill_upper, key_bias=key_bias, first_visible=first_visible)
        if zero_planes is not None:
            # (a mask under which some row sees nothing: that row's NaN becomes zeros, as behind the reference's masked_fill
            # ahead of its post-softmax conv - and the stored probabilities give it a zero gradient.  Either the mask's uint8
            # visibility planes, or for a band mask an int32 (B,S) array that is p + 1 for such a row p and 0 elsewhere)
            if zero_planes.dtype == torch.int32:
                if ops.band_zero_(p, zero_planes) is None:
                    raise RuntimeError("band masks need 16-bit scores of a length that is a multiple of 8")
            else:
                ops.mask_fill(p, zero_planes, False, causal, out=p)
        ctx.save_for_backward(x if weight is not None else None, weight, p)
        ctx.causal, ctx.group_size, ctx.grad_fill_upper = causal, group_size, grad_fill_upper
        return p

    @staticmethod
    def backward(ctx, grad_output):
        x, weight, p = ctx.saved_tensors
        # the head mixing's gradient kernels never read above the diagonal; whoever takes the gradient we return might
        ds = ops.softmax_bwd(p, grad_output.to(p.dtype), ctx.causal,
                             fill_upper=weight is None and ctx.grad_fill_upper)
        if weight is None:
            return ds, None, None, None, None, None, None, None, None
        dx = dw = None
        if ctx.needs_input_grad[0]:
            dx = ops.headmix_bwd_input(ds, weight, ctx.causal, ctx.group_size, fill_upper=ctx.grad_fill_upper)
        if ctx.needs_input_grad[1]:
            dw = ops.headmix_bwd_weight(x, ds, ctx.causal)
            if ctx.group_size:
                blk = torch.arange(weight.shape[0], device=weight.device) // ctx.group_size
                dw = dw * (blk[:, None] == blk[None, :])
            dw = dw.to(weight.dtype)
        return dx, dw, None, None, None, None, None, None, None


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


@dataclass(frozen=True)
class WeightStructure:
    """What the glue may assume about the four weights (all False / None = nothing)."""
    pre_head_identity: bool = False
    pre_head_group: Optional[int] = None      # None = dense
    post_conv_identity: bool = False
    post_head_identity: bool = False
    post_head_group: Optional[int] = None


_DENSE = WeightStructure()


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
        # layout of the score tensors between the kernels of the inference route: "auto" = triangular where all three
        # kernels know it, "planes" = (B,H,S,S) always (MTA_SCORE_LAYOUT=planes in the environment: the same, for
        # comparisons)
        self.score_layout = "planes" if os.environ.get("MTA_SCORE_LAYOUT") == "planes" else "auto"
        # "dense": assume nothing; "declared": use self._declared; "probe": look at the weights on every call
        self.weight_structure = "dense"
        self._declared = WeightStructure()
        self.register_load_state_dict_post_hook(lambda module, incompatible: module.assume_dense_weights())

    # ------------------------------------------------------------------ forward
    def _mark(self, name: str) -> None:
        if self._stage_hook is not None:
            self._stage_hook(name)


    def forward(self, xq, xk, xv, mask, chunk_start_ids):
        assert chunk_start_ids is None, "MTAAttentionTriton does not support chunked attention"
        wants_grad = torch.is_grad_enabled() and (xq.requires_grad or xk.requires_grad or xv.requires_grad
                                                  or any(p.requires_grad for p in self.parameters()))
        if self.use_mask:
            return self._forward_with_mask(xq, xk, xv, mask, wants_grad)
        if wants_grad:
            return self._forward_stagewise(xq, xk, xv)
        return self._forward_fused(xq, xk, xv)

    def _forward_fused(self, xq, xk, xv, key_bias=None, first_visible=None, empty_rows=None):
        """Inference route (module docstring).  ``key_bias``: fp32 (B,Sk), added to the mixed scores ahead of the
        softmax -- the caller has zeroed the K and V rows of the keys it hides.  ``first_visible``: int32 (B,S), a band
        mask (row p sees the keys first_visible[p] .. p): applied to the scores inside the first kernel and as -inf
        inside the softmax kernel, and behind a post-softmax conv that is not the identity the hidden stretch of every row
        is zeroed again; the caller has checked that the first kernel exists.  ``empty_rows``: bool (B,S) or None, the
        rows of the band that see no key (first_visible[p] = p + 1).  Their scores enter the conv as 0 like any hidden
        score; the softmax leaves NaN in them, which the reference replaces by zeros ahead of its post-softmax conv
        (mta_attention_triton.py:81): here those rows of the probabilities are cleared ahead of a post-softmax conv
        that is not the identity, and their rows of the output, where nothing else would, at the end."""
        head_dim = xq.size(-1)
        # the reference multiplies by rsqrt(tensor(head_dim)), an fp32 scalar (mta_attention_triton.py:69-71)
        scale = float(torch.rsqrt(torch.tensor(float(head_dim))))
        st = self._current_structure()
        w_pre, w_post = self.wpsm_triton.weight, self.wposm_triton.weight
        g_pre = st.pre_head_group or self.n_heads
        g_post = st.post_head_group or self.n_heads
        w1 = None if st.pre_head_identity else w_pre
        w2 = None if st.post_head_identity else w_post
        if w1 is None:
            g_pre = 1
        if w2 is None:
            g_post = 1
        post_conv_identity = st.post_conv_identity
        n_keys = xk.size(-2)
        g_both = _lcm(g_pre, g_post)
        # (the matrix-core variant for groups of 16 takes a key bias or a band mask in its row-list form only)
        row_plain = key_bias is None and first_visible is None
        masks_ok = lambda group: row_plain or group <= _FUSED_MAX_GROUP or (
            group == _FUSED_MFMA_GROUP and os.environ.get("MTA_MIX16_NO_ROW_LISTS") != "1")
        one_pass = post_conv_identity and _one_pass_group(g_both, xq.dtype, n_keys, w1, w2) and masks_ok(g_both)
        # the last stage may leave the upper triangle unwritten only if our own P V kernel consumes it
        own_pv = (xq.size(-2) == xk.size(-2) and xq.dtype == xv.dtype
                  and ops.causal_pv_supported(xq.dtype, xq.size(-2), xv.size(-1)))

        # Three kernels with nothing elementwise between them: the two score tensors are nobody else's business, and they
        # travel in the triangular layout (what lies on and below the diagonal only, the rows a workgroup of the softmax
        # stage reads side by side): half the footprint, and every stage streams memory in longer runs.
        if (self.score_layout != "planes" and self.causal and one_pass and own_pv
                and not (self.training and self.dropout > 0) and g_both in (2, 4, 8, 16)
                and (key_bias is None or (key_bias.is_contiguous() and key_bias.data_ptr() % 16 == 0))
                and ops.tri_route_supported(xq, xk, self.mta_conv_triton.weight, g_both, w1, w2, first_visible is not None,
                                            key_bias=key_bias is not None)):
            self._mark("qk_conv")
            scores = ops.qk_conv_tri(xq, xk, self.mta_conv_triton.weight, scale, g_both, first_visible=first_visible)
            self._mark("mix_softmax_mix")
            scores = ops.headmix_softmax_tri(scores, w1, w2, xq.size(0), self.n_heads, n_keys, g_both,
                                             first_visible=first_visible, key_bias=key_bias)
            self._mark("pv")
            output = ops.causal_pv_tri(scores, xv, g_both, first_visible=first_visible)
            if empty_rows is not None:
                output.masked_fill_(empty_rows[:, None, :, None], 0)
            self._mark("end")
            return output.transpose(1, 2)

        # QK^T -> *1/sqrt(d) -> conv: one kernel when it exists for this dtype / size, else GEMM + conv
        scores = None
        # (dense groups of 16 heads ahead of a post-softmax conv: the first score tensor still travels in the triangular
        # layout, the softmax stage hands the conv (B,H,S,S) planes)
        tri_first = (self.score_layout != "planes" and self.causal and not one_pass and g_pre == 16 and masks_ok(16)
                     and w1 is not None and not (post_conv_identity and w2 is None and not own_pv)
                     and (key_bias is None or key_bias.is_contiguous())
                     and ops.tri_route_supported(xq, xk, self.mta_conv_triton.weight, 16, w1, None, first_visible is not None,
                                                 out_planes=True, key_bias=key_bias is not None))
        if tri_first:
            self._mark("qk_conv")
            scores = ops.qk_conv_tri(xq, xk, self.mta_conv_triton.weight, scale, 16, first_visible=first_visible)
        elif ops.qk_conv_supported(xq, xk, self.mta_conv_triton.weight):
            self._mark("qk_conv")
            scores = ops.qk_conv(xq, xk, self.mta_conv_triton.weight, self.causal, scale, fill_upper=False,
                                 first_visible=first_visible)
        if scores is None:
            assert first_visible is None, "the band mask needs the one-kernel first stage"
            self._mark("qk")
            scores = torch.matmul(xq, xk.transpose(2, 3))
            self._mark("conv_pre")
            scores = ops.conv2d_causal(scores, self.mta_conv_triton.weight, self.causal, in_scale=scale)

        if one_pass:
            self._mark("mix_softmax_mix")
            scores = ops.headmix_softmax(scores, w1, w2, self.causal, group_size=g_both,
                                         fill_upper=not own_pv, key_bias=key_bias, first_visible=first_visible)
        else:
            if tri_first:
                self._mark("mix_softmax")
                scores = ops.headmix_softmax_tri(scores, w1, None, xq.size(0), self.n_heads, n_keys, g_pre, out_planes=True,
                                                 first_visible=first_visible, key_bias=key_bias)
            elif _one_pass_group(g_pre, xq.dtype, n_keys, w1) and masks_ok(g_pre):
                self._mark("mix_softmax")
                scores = ops.headmix_softmax(scores, w1, None, self.causal, group_size=g_pre, key_bias=key_bias,
                                             first_visible=first_visible,
                                             fill_upper=post_conv_identity and w2 is None and not own_pv)
            else:
                self._mark("mix_pre")
                fill = float("-inf") if self.causal else 0.0
                # (the softmax kernel that follows never reads above the diagonal)
                scores = ops.headmix(scores, w_pre, self.causal, fill, group_size=g_pre, fill_upper=False)
                self._mark("softmax")
                scores = ops.headmix_softmax(scores, None, None, self.causal, key_bias=key_bias,
                                             first_visible=first_visible,
                                             fill_upper=post_conv_identity and w2 is None and not own_pv)
            if empty_rows is not None and not post_conv_identity:
                # (the rows that see nothing, NaN out of the softmax: zeros into the conv, whole rows up to the diagonal)
                rows_all = torch.arange(1, n_keys + 1, device=empty_rows.device, dtype=torch.int32)
                if ops.band_zero_(scores, torch.where(empty_rows, rows_all[None, :], 0).to(torch.int32)) is None:
                    raise RuntimeError("band masks need 16-bit scores of a length that is a multiple of 8")
            done = None
            # conv and mix in one pass, the conv result never written: taken where it measures at least as fast as the
            # two kernels (mixing groups of up to 4 heads, kernel sizes with a vector-staged instance: 3x3, 7x7)
            ks = tuple(self.mta_conv_after_sm_triton.weight.shape[1:])
            conv_w = self.mta_conv_after_sm_triton.weight
            mix16 = (g_post == 16 and ks in _CONV_MIX16_SIZES and scores.dtype in (torch.bfloat16, torch.float16)
                     and conv_w.dtype == scores.dtype and w_post.dtype == scores.dtype and n_keys % 8 == 0)
            # (under a band mask the conv's result is zeroed at the hidden positions ahead of the mixing, as the reference
            # does: two kernels with that step between them)
            if first_visible is None and not post_conv_identity and w2 is not None and (
                    (g_post <= _CONV_MIX_MAX_GROUP and ks in _CONV_MIX_SIZES) or mix16):
                self._mark("conv_mix_post")
                done = ops.conv2d_headmix(scores, self.mta_conv_after_sm_triton.weight, w_post, self.causal,
                                          group_size=g_post, fill_upper=not own_pv)
            if done is not None:
                scores = done
            else:
                # neither our head mixing nor our P V reads above the diagonal: whoever feeds them need not write there
                if not post_conv_identity:
                    self._mark("conv_post")
                    scores = ops.conv2d_causal(scores, self.mta_conv_after_sm_triton.weight, self.causal,
                                               fill_upper=w2 is None and not own_pv)
                    if first_visible is not None:
                        # the conv has spread probability into columns the rows do not see
                        # (mta_attention_triton.py:82-83: torch.where(mask == -inf, 0.0, scores))
                        if ops.band_zero_(scores, first_visible) is None:
                            raise RuntimeError("band masks need 16-bit scores of a length that is a multiple of 8")
                if w2 is not None:
                    self._mark("mix_post")
                    scores = ops.headmix(scores, w_post, self.causal, 0.0, group_size=g_post, fill_upper=not own_pv)

        scores = F.dropout(scores, p=self.dropout, training=self.training)
        self._mark("pv")
        output = ops.causal_pv(scores, xv, self.causal, first_visible=first_visible) if own_pv else None
        if output is None:
            output = torch.matmul(scores, xv)
        if empty_rows is not None:
            output.masked_fill_(empty_rows[:, None, :, None], 0)
        self._mark("end")
        return output.transpose(1, 2)

    def _forward_stagewise(self, xq, xk, xv, key_bias=None, first_visible=None, mask_planes=None, mask_additive=None,
                           mask_empty_rows=False, band_empty_rows=None):
        """The reference's own sequence of operators (mta_attention_triton.py:68-92), each differentiable: taken
        whenever a gradient may be asked for.  No weight structure is assumed here, so every entry of the four
        weights receives its gradient.

        ``key_bias`` (fp32 (B,Sk), 0 / -inf per key, or finite values of a 2-D additive mask): "causal rule + hidden
        keys" under use_mask (mta_attention_triton.py:72-73, 77, 81-83).  The K and V rows of the hidden keys are zeroed
        (differentiably: those rows receive no gradient, as in the reference, whose masked_fill / where cut it): the
        scores of their columns then enter the pre-softmax conv as 0, the bias hides them from the softmax, and what the
        post-softmax conv writes into their columns meets zero V rows - and receives a zero gradient from them.

        ``first_visible`` (int32 (B,S)): a band mask, row p sees the keys first_visible[p] .. p.  Applied where the
        reference applies the mask tensor: to the scores ahead of the pre-softmax conv (inside the scores kernel), as
        -inf inside the softmax kernel, and as zeros behind the post-softmax conv; the caller has checked that the
        kernels this needs exist (``_band_training_supported``).

        ``mask_planes`` (uint8 (1|B, 1|H, S, S), non-zero = attend): a 0 / -inf mask of arbitrary content.  The three
        elementwise mask steps of the reference run as in-place passes between the operators (``_MaskFill``, and inside
        ``_ScaledScoresConv``); head mixing and softmax run as two kernels, the mask goes between them."""
        if key_bias is not None:
            hidden = (key_bias == float("-inf"))[:, None, :, None]
            xk = xk.masked_fill(hidden, 0)
            xv = xv.masked_fill(hidden, 0)
        scale = float(torch.rsqrt(torch.tensor(float(xq.size(-1)))))
        scores = _ScaledScoresConv.apply(xq, xk, self.mta_conv_triton.weight, scale, self.causal, self._mark,
                                         first_visible, mask_planes)
        group = self.wpsm_triton.group_size
        w_pre = self.wpsm_triton.weight
        # Between two of these stages nothing reads above the diagonal (causal kernels never do, in either direction),
        # so nothing is written there: only the last stage's output, which torch's GEMM reads in full, and the score
        # gradient that goes into torch's GEMMs (inside _ScaledScoresConv) are filled.
        lower = not self.causal   # value of the fill flags: False (leave alone) when causal
        # (band_empty_rows: bool (B,S), the rows of the band mask that see no key: their probabilities are cleared)
        zero_rows = mask_planes if mask_empty_rows else None
        if band_empty_rows is not None:
            rows_all = torch.arange(1, xk.size(-2) + 1, device=xq.device, dtype=torch.int32)
            zero_rows = torch.where(band_empty_rows, rows_all[None, :], 0).to(torch.int32).contiguous()
        g_eff = group or self.n_heads
        # (the matrix-core variant for groups of 16 takes a key bias in its row-list form only)
        bias_ok = (key_bias is None and first_visible is None) or g_eff <= _FUSED_MAX_GROUP or (
            g_eff == _FUSED_MFMA_GROUP and os.environ.get("MTA_MIX16_NO_ROW_LISTS") != "1")
        if _one_pass_group(g_eff, scores.dtype, xk.size(-2), w_pre) and bias_ok and mask_planes is None:
            self._mark("mix_softmax")
            scores = _MixSoftmax.apply(scores, w_pre, self.causal, group, lower, lower, key_bias, first_visible, zero_rows)
        else:
            self._mark("mix_pre")
            scores = TritonLinearHeadFunction.apply(scores, w_pre, self.wpsm_triton.causal, self.wpsm_triton.output_value,
                                                    group, lower, lower)
            if mask_planes is not None:
                self._mark("mask")
                if mask_additive is None:
                    scores = _MaskFill.apply(scores, mask_planes, True, self.causal)
                else:   # (finite values besides 0: the mask in the scores' dtype is added)
                    scores = _MaskAdd.apply(scores, mask_additive, self.causal)
            self._mark("softmax")
            scores = _MixSoftmax.apply(scores, None, self.causal, None, lower, lower, key_bias, first_visible, zero_rows)
        self._mark("conv_post")
        scores = Conv2dTritonFunction.apply(scores, self.mta_conv_after_sm_triton.weight, self.causal, lower, lower)
        if first_visible is not None:
            scores = _BandZero.apply(scores, first_visible)
        if mask_planes is not None:
            self._mark("mask")
            scores = _MaskFill.apply(scores, mask_planes, False, self.causal)
        self._mark("mix_post")
        post = self.wposm_triton
        # the last stage's output is read by P V: in full by the library GEMM, on and below the diagonal by our kernels
        lower_pv = (self.causal and post.causal and scores.dtype == xv.dtype
                    and _lower_products_supported(xv, scores.size(-1)) and scores.size(-2) == scores.size(-1))
        scores = TritonLinearHeadFunction.apply(scores, post.weight, post.causal, post.output_value, post.group_size,
                                                not lower_pv, lower)
        scores = F.dropout(scores, p=self.dropout, training=self.training)
        self._mark("pv")
        # (the gradient with respect to the probabilities goes back into the head mixing's gradient kernels, through the
        # dropout's elementwise mask at most: nothing there reads above the diagonal when causal)
        assert first_visible is None or lower_pv
        output = _ProbsTimesValues.apply(scores, xv, lower_pv, first_visible)
        self._mark("end")
        return output.transpose(1, 2)

    # ------------------------------------------------------------------ weight structure
    def _current_structure(self) -> "WeightStructure":
        if self.weight_structure == "dense":
            return _DENSE
        if self.weight_structure == "declared":
            return self._declared
        if self.weight_structure == "probe":
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError('weight_structure="probe" reads the probe result back on every call and cannot run '
                                   "under stream capture: call infer_weight_structure() before capturing instead")
            return self._probe_now()
        raise ValueError(f"weight_structure must be 'dense', 'declared' or 'probe', got {self.weight_structure!r}")

    def _probe_now(self) -> "WeightStructure":
        pre_eye, g_pre, post_eye, g_post, conv_eye = ops.probe_mta_weights(
            self.wpsm_triton.weight, self.wposm_triton.weight, self.mta_conv_after_sm_triton.weight)
        return WeightStructure(pre_head_identity=pre_eye, pre_head_group=g_pre, post_conv_identity=conv_eye,
                               post_head_identity=post_eye, post_head_group=g_post)

    def infer_weight_structure(self) -> "WeightStructure":
        """Look at the current weights once (device-side probe, one small read back) and keep the result for
        all later calls.  Call again after the weights change; see the module docstring."""
        self._declared = self._probe_now()
        self.weight_structure = "declared"
        return self._declared

    def declare_weight_structure(self, pre_head_identity: bool = False, pre_head_group: Optional[int] = None,
                                 post_conv_identity: bool = False, post_head_identity: bool = False,
                                 post_head_group: Optional[int] = None) -> "WeightStructure":
        """State the structure of the weights without looking at them: ``*_identity`` = that weight is exactly
        the identity (head weights) / the pass-through tap at [R-1, S//2] (post-softmax conv);
        ``*_head_group`` = G such that the head weight is zero outside its GxG diagonal blocks."""
        for g in (pre_head_group, post_head_group):
            if g is not None and (g <= 0 or self.n_heads % g):
                raise ValueError(f"head group {g} does not divide n_heads={self.n_heads}")
        self._declared = WeightStructure(pre_head_identity, pre_head_group, post_conv_identity, post_head_identity,
                                         post_head_group)
        self.weight_structure = "declared"
        return self._declared

    def assume_dense_weights(self) -> None:
        """Back to the default: nothing is assumed about the weights."""
        self._declared = WeightStructure()
        self.weight_structure = "dense"

    def _forward_with_mask(self, xq, xk, xv, mask, wants_grad=True):
        """use_mask=True: an explicit additive mask tensor drives the masking (mta_attention_triton.py:63-64,
        77-83, 96-98); the kernels still apply their own causal rule when ``causal`` is set.

        These masks never become a (B,H,S,S) tensor here (causal module, inference and training): no mask at all, which
        the reference turns into the causal rule the kernels apply anyway; a 2-D key mask, which the reference turns into
        "causal rule + one value per key" (mta_attention_triton.py:118-122); a 4-D mask that says the same per batch
        entry (key padding for B > 1, which the reference's 2-D form cannot express); and a 4-D band mask.  A hidden
        key's scores enter the pre-softmax conv as 0 -- which is what a zero K row produces -- its mixed score gets -inf
        ahead of the softmax (the kernel's per-key bias), its probability is 0, and whatever the post-softmax conv writes
        into its column, which the reference zeroes, meets a zero V row.  A ``causal=False`` module knows the hidden-keys
        form (the same keys hidden from every row).  Any other 4-D mask over square scores whose length is a multiple of
        8 is read as a byte per position by three mask passes between the single-stage kernels; what is left takes the
        reference's own steps, at the end of this function."""
        if self.causal and xq.size(-2) == xk.size(-2):
            # (with a gradient wanted: the same masks through the differentiable operators)
            hidden_keys = self._forward_stagewise_hidden_keys if wants_grad else self._forward_hidden_keys
            if not isinstance(mask, torch.Tensor):
                return self._forward_stagewise(xq, xk, xv) if wants_grad else self._forward_fused(xq, xk, xv)
            if mask.dim() == 2 and xq.size(0) == 1:
                assert mask.size(0) == xq.size(0)
                if mask.dtype == torch.bool:
                    bias = torch.where(mask, 0.0, float("-inf")).to(torch.float32)
                else:
                    bias = mask.type(xq.dtype).to(torch.float32)   # the reference adds it in the I/O dtype
                return hidden_keys(xq, xk, xv, bias.contiguous())
            # a 4-D mask, the same for all heads, of one of two forms goes into the kernels without a (B,H,S,S) tensor:
            # "causal rule + hidden keys" per batch entry (key padding: a key bias and zeroed K and V rows, as for the
            # 2-D mask above) and "row p sees the keys first[p] .. p" (sliding windows, packed documents: one int32 per
            # batch entry and row)
            if mask.dim() == 4:
                kind, what = self._structured_mask(mask, xq.size(0), xq.size(-2))
                if kind == "keys":
                    return hidden_keys(xq, xk, xv, what)
                if kind == "band" and ops.qk_conv_supported(xq, xk, self.mta_conv_triton.weight):
                    empty_rows = self._band_empty_rows(mask)
                    if not wants_grad:
                        return self._forward_fused(xq, xk, xv, first_visible=what, empty_rows=empty_rows)
                    if self._band_training_supported(xq, xk, xv):
                        return self._forward_stagewise(xq, xk, xv, first_visible=what, band_empty_rows=empty_rows)
        elif (not self.causal and isinstance(mask, torch.Tensor) and mask.dim() == 4 and xq.size(-2) == xk.size(-2)):
            # no causal rule and a mask that hides the same keys from every row (key padding of an encoder batch): the same
            # key bias and zeroed K and V rows, through the kernels' non-causal form
            kind, what = self._structured_mask(mask, xq.size(0), xq.size(-2))
            if kind == "keys":
                if wants_grad:
                    return self._forward_stagewise(xq, xk, xv, key_bias=what)
                return self._forward_hidden_keys(xq, xk, xv, what)
        if (isinstance(mask, torch.Tensor) and mask.dim() == 4 and xq.size(-2) == xk.size(-2) and xk.size(-2) % 8 == 0):
            planes, additive, empty_rows = self._mask_planes(mask, xq.size(0), xq.size(-2))
            if additive is not None:   # (the reference adds the mask in the scores' dtype)
                additive = additive.to(xq.dtype).contiguous()
                if additive.data_ptr() % 16 != 0:
                    planes = None
            if planes is not None:
                if wants_grad:
                    return self._forward_stagewise(xq, xk, xv, mask_planes=planes, mask_additive=additive,
                                                   mask_empty_rows=empty_rows)
                return self._forward_mask_planes(xq, xk, xv, planes, additive, empty_rows)
        mask = self._update_mask(mask=mask, bsz=xq.size(0), xq=xq, xk_size=xk.size(-2))
        scale = float(torch.rsqrt(torch.tensor(float(xq.size(-1)))))  # a host scalar: the product stays one vectorised pass
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

    def _forward_mask_planes(self, xq, xk, xv, visible, additive=None, empty_rows=False):
        """Inference under a boolean or additive mask of arbitrary content - holes, planes per head - given as uint8
        visibility planes (1|B, 1|H, S, S), and for an additive mask with finite values besides 0 as that mask in the
        scores' dtype as well (added ahead of the softmax in place of the -inf fill): the reference's sequence
        (mta_attention_triton.py:68-92) on the single-stage kernels, with its three elementwise mask steps as one in-place pass each that reads a byte per position
        (``mta_mask_fill_fwd``): no mask tensor in the score dtype, no boolean copy of it, no fp32 copy of the scores,
        and under the causal rule nothing above the diagonal is computed, masked or written."""
        cz = self.causal
        fu = not cz   # (fill flags of the causal kernels: nothing above the diagonal is anybody's business)
        scale = float(torch.rsqrt(torch.tensor(float(xq.size(-1)))))
        n_keys = xk.size(-2)
        own_pv = cz and xq.dtype == xv.dtype and ops.causal_pv_supported(xq.dtype, n_keys, xv.size(-1))
        self._mark("qk")
        scores = _lower_scores(xq, xk) if cz else None
        if scores is None:
            scores = torch.matmul(xq, xk.transpose(2, 3))
        self._mark("mask")
        if ops.mask_fill(scores, visible, False, cz, out=scores) is None:
            raise RuntimeError("mask planes need a number of keys that is a multiple of 8")
        self._mark("conv_pre")
        scores = ops.conv2d_causal(scores, self.mta_conv_triton.weight, cz, in_scale=scale, fill_upper=fu)
        # (a declared or inferred weight structure: identity stages are skipped - the probabilities are 0 at the hidden
        # positions already, so without a post-softmax conv its mask pass goes too - and block-diagonal head weights are
        # applied block by block)
        st = self._current_structure()
        if not st.pre_head_identity:
            self._mark("mix_pre")
            scores = ops.headmix(scores, self.wpsm_triton.weight, cz, float("-inf") if cz else 0.0,
                                 group_size=st.pre_head_group, fill_upper=fu)
        self._mark("mask")
        if additive is None:
            ops.mask_fill(scores, visible, True, cz, out=scores)
        elif ops.mask_add(scores, additive, cz, out=scores) is None:
            raise RuntimeError("mask planes need a number of keys that is a multiple of 8")
        self._mark("softmax")
        last = st.post_conv_identity and st.post_head_identity   # (the softmax's output goes to P V)
        scores = ops.headmix_softmax(scores, None, None, cz, fill_upper=(not own_pv) if last else fu)
        if empty_rows:
            # a row that sees nothing comes out of the softmax as NaN; the reference's masked_fill ahead of its
            # post-softmax conv turns it into zeros (everywhere else the hidden positions hold 0 already)
            self._mark("mask")
            ops.mask_fill(scores, visible, False, cz, out=scores)
        if not st.post_conv_identity:
            self._mark("conv_post")
            scores = ops.conv2d_causal(scores, self.mta_conv_after_sm_triton.weight, cz,
                                       fill_upper=(not own_pv) if st.post_head_identity else fu)
            self._mark("mask")
            ops.mask_fill(scores, visible, False, cz, out=scores)
        if not st.post_head_identity:
            self._mark("mix_post")
            scores = ops.headmix(scores, self.wposm_triton.weight, cz, 0.0, group_size=st.post_head_group,
                                 fill_upper=not own_pv)
        scores = F.dropout(scores, p=self.dropout, training=self.training)
        self._mark("pv")
        output = ops.causal_pv(scores, xv, True) if own_pv else None
        if output is None:
            output = torch.matmul(scores, xv)
        self._mark("end")
        return output.transpose(1, 2)

    def _band_training_supported(self, xq, xk, xv) -> bool:
        """Whether the differentiable route takes a band mask: 16-bit data of one dtype, a length the in-place zeroing
        kernel takes, and the lower-triangle products (P V and its gradients, the recomputed raw scores) as kernels."""
        s = xk.size(-2)
        return (xq.dtype in (torch.bfloat16, torch.float16) and xq.dtype == xk.dtype == xv.dtype
                and xq.shape == xk.shape and s % 8 == 0 and _lower_products_supported(xv, s)
                and _lower_products_supported(xq, s)
                and all(w.dtype == xq.dtype for w in (self.mta_conv_triton.weight, self.mta_conv_after_sm_triton.weight,
                                                      self.wpsm_triton.weight, self.wposm_triton.weight)))

    def _forward_stagewise_hidden_keys(self, xq, xk, xv, bias):
        return self._forward_stagewise(xq, xk, xv, key_bias=bias)

    def _forward_hidden_keys(self, xq, xk, xv, bias):
        """The fused route under "causal rule + one additive value per (batch entry, key)" (``bias``: fp32 (B,S)).  The K
        rows of hidden keys (-inf) are zeroed: their scores then enter the pre-softmax conv as 0.  Their probabilities
        are 0; a post-softmax conv that is not the identity writes into their columns all the same, which the reference
        zeroes again - here those columns meet zeroed V rows instead."""
        hidden = (bias == float("-inf"))[:, None, :, None]
        if not self._current_structure().post_conv_identity:
            xv = xv.masked_fill(hidden, 0)
        return self._forward_fused(xq, xk.masked_fill(hidden, 0), xv, key_bias=bias)

    def _structured_mask(self, mask, bsz: int, s: int):
        """What a 4-D ``mask`` (bool with True = attend, or additive with 0 / -inf; one plane for all heads) amounts to
        together with the causal rule (a module with ``causal=False``: on its own, and only the first form):
          ("keys", bias)   every row sees the kept keys up to itself and key 0 is kept: fp32 (B,S), 0 / -inf per key;
          ("band", first)  row p sees exactly the keys first[p] .. p, or none at all (first[p] = p + 1): int32 (B,S);
          (None, None)     anything else (per-head planes, holes that differ between rows, other finite values, a row
                           that sees nothing).
        A few reductions over the mask and one read back; the answer for the last mask object seen is kept while its
        version does not change."""
        if mask.size(0) not in (1, bsz) or mask.size(-2) != s or mask.size(-1) != s or mask.size(1) not in (1, self.n_heads):
            return None, None
        key = (mask._version, bsz)
        cached = getattr(self, "_mask_cache", None)   # (the mask object itself is kept: its identity cannot be reused)
        if cached is not None and cached[0] is mask and cached[1] == key:
            return cached[2]
        answer, empty_rows = (None, None), None
        plane = mask[:, 0]
        same_heads = mask.size(1) == 1 or bool((mask == mask[:, :1]).all())
        if mask.dtype == torch.bool:
            visible = plane
        else:
            visible = plane == 0
            if not bool(((plane == float("-inf")) | visible).all()):
                visible = None   # other finite values: not a 0 / -inf mask
        if same_heads and visible is not None and not self.causal:
            # no causal rule: "hidden keys" means every row sees the same keys, and at least one
            keep = visible[:, 0, :]
            if bool((visible == keep[:, None, :]).all()) and bool(keep.any(-1).all()):
                bias = torch.where(keep, 0.0, float("-inf")).to(torch.float32).expand(bsz, s).contiguous()
                answer = ("keys", bias)
        elif same_heads and visible is not None:
            rows = torch.arange(s, device=mask.device)
            lower = rows[None, :] <= rows[:, None]
            visible = visible & lower
            keep = visible[:, -1, :]                       # what the last row sees: every kept key
            if bool((visible == (keep[:, None, :] & lower)).all()) and bool(keep[:, 0].all()):
                bias = torch.where(keep, 0.0, float("-inf")).to(torch.float32).expand(bsz, s).contiguous()
                answer = ("keys", bias)
            else:
                count = visible.sum(-1)
                lead = visible.int().argmax(-1)
                empty = count == 0      # rows that see no key (the padding of a left-padded batch): first[p] = p + 1
                if bool((empty | (count == rows[None, :] - lead + 1)).all()):
                    first = torch.where(empty, rows[None, :] + 1, lead)
                    answer = ("band", first.to(torch.int32).expand(bsz, s).contiguous())
                    if bool(empty.any()):
                        empty_rows = empty.expand(bsz, s).contiguous()
        self._mask_cache = (mask, key, answer, empty_rows)
        return answer

    def _band_empty_rows(self, mask):
        """bool (B,S): the query rows of the band mask last classified that see no key at all, or None if every row sees
        one."""
        cached = getattr(self, "_mask_cache", None)
        return cached[3] if cached is not None and cached[0] is mask else None

    def _mask_planes(self, mask, bsz: int, s: int):
        """(planes, additive, empty_rows) of a 4-D mask (1|B, 1|H, S, S) that is none of the forms ``_structured_mask``
        knows: the mask as a byte per position (uint8, non-zero = attend: a boolean mask as it is, an additive one as "not
        -inf"); the mask itself if it is additive with finite values besides 0 (else None); and whether some query row
        sees no key at all (the padding rows of a left-padded batch) - the softmax of such a row is NaN, which the
        reference replaces by zeros ahead of its post-softmax conv (mta_attention_triton.py:81), and so does the route
        then.  (None, None, False) for a mask of another shape.
        Kept for the last mask object seen while its version does not change (for an additive mask the planes are a
        tensor of their own, a byte per mask element)."""
        if mask.size(0) not in (1, bsz) or mask.size(-2) != s or mask.size(-1) != s or mask.size(1) not in (1, self.n_heads):
            return None, None, False
        cached = getattr(self, "_planes_cache", None)
        if cached is not None and cached[0] is mask and cached[1] == mask._version:
            return cached[2]
        if mask.dtype == torch.bool:
            visible, additive = mask.contiguous(), None
        else:
            blocked = mask == float("-inf")
            finite = not bool((blocked | (mask == 0)).all())
            visible, additive = ~blocked, (mask if finite else None)
        seen = visible.tril() if self.causal else visible     # (the kernels apply the causal rule on top of the mask)
        empty_rows = not bool(seen.any(-1).all())
        answer = (visible.view(torch.uint8), additive, empty_rows)
        self._planes_cache = (mask, mask._version, answer)
        return answer

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
        self.assume_dense_weights()

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
        self.assume_dense_weights()


def _lcm(a: int, b: int) -> int:
    import math
    return a * b // math.gcd(a, b)


__all__ = ["MTAAttentionTriton", "MTAConfig", "WeightStructure"]
