"""CPU oracle for the Multi-Token-Attention forward path.  TEST INFRASTRUCTURE ONLY.

This file restates, with the same torch library routines the reference calls, what
the reference's PyTorch modules compute.  It is the checker the HIP kernels are
compared with; nothing in the product package may import it.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` use it.

Every function is device-agnostic (runs on the CPU) and cites the reference lines it
follows.  How each one is pinned (see tests/test_oracle.py):

* ``depthwise_conv`` / ``mta_convolution``: brute-force nested loops in C
  (oracle/mta_oracle.c), scipy.signal.correlate2d per plane, delta-kernel == shift,
  identity tap == tril(x) bit-exact, linearity.
* ``head_linear``: einsum against nested C loops, W=I pass-through, permutation W.
* ``mta_forward``: all-identity weights == causal scaled-dot-product attention,
  row 0 closed form, stage-by-stage equality with the C restatement; its tensor-mask
  branch (bool, (1,Sk) key mask, (1,1,S,S) additive) against the C restatement given
  the same additive mask; ``mta_forward_rows`` (slab form) == full form.
* ``depthwise_conv_grads`` / ``head_linear_grads`` (autograd through the two operators):
  gradcheck in fp64, the C restatement of the reference's backward kernels, adjoint
  identities.
* ``conv_attention_forward``: identity tap == causal SDPA, C restatement, equality
  with the composition of the pinned stages, slab form == full form.

The reference ships no golden vectors or tests for this path; the fixtures under
tests/golden/ are regression vectors written by this oracle after the pins above.
"""
from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn.functional as F

NEG_INF = float("-inf")


# ---------------------------------------------------------------------------
# masks
# ---------------------------------------------------------------------------
def update_mask(mask, bsz: int, n_heads: int, xq: torch.Tensor, xk_size: int) -> torch.Tensor:
    """Additive mask of shape (B,H,Sq,Sk): 0 where attended, -inf where not.

    Follows mta_attention_pytorch.py:114-137 (same rules as
    mta_attention_triton.py:106-127): a non-tensor mask means plain causal; a bool
    mask maps True->0 / False->-inf; a 2-D (B,Sk) key mask is broadcast over heads
    and query rows and then made causal; a (1,1,Sq,Sk) mask is repeated.
    """
    sq = xq.size(-2)
    if not isinstance(mask, torch.Tensor):
        m = torch.full((sq, xk_size), NEG_INF, device=xq.device)
        m = torch.triu(m, diagonal=1).type_as(xq)
        return m.repeat(bsz, n_heads, 1, 1)
    if mask.dtype == torch.bool:
        mask = torch.where(mask, 0.0, NEG_INF).to(xq.dtype)
    if mask.dtype != xq.dtype:
        mask = mask.type(xq.dtype)
    if mask.dim() == 2:
        assert mask.size(0) == bsz
        mask = mask.repeat(1, n_heads, sq, 1)
        mi, mj = torch.triu_indices(sq, xk_size, offset=1)
        mask[:, :, mi, mj] = NEG_INF
    elif mask.size(0) == 1 and mask.size(1) == 1:
        mask = mask.repeat(bsz, n_heads, 1, 1)
    return mask


# ---------------------------------------------------------------------------
# stage: key-query convolution
# ---------------------------------------------------------------------------
def mta_convolution(scores: torch.Tensor, mask: torch.Tensor, kernel: torch.Tensor,
                    pad_key: str = "both") -> torch.Tensor:
    """Depthwise conv over the (query,key) plane of each head, masked taps read as 0.

    Follows mta_attention_pytorch.py:85-112.  ``kernel`` is (H,1,R,S).  Padding is
    R-1 rows on top only; key padding "both" = (S-1)//2 on each side, "left"/"right"
    = S-1 on that side.  No mask is applied to the OUTPUT here.
    """
    scores = torch.where(mask == NEG_INF, 0.0, scores)
    n_heads, head_sz, qdim, kdim = kernel.shape
    if pad_key == "left":
        padded = F.pad(scores, (kdim - 1, 0, qdim - 1, 0), value=0.0)
    elif pad_key == "right":
        padded = F.pad(scores, (0, kdim - 1, qdim - 1, 0), value=0.0)
    elif pad_key == "both":
        assert (kdim - 1) % 2 == 0
        padded = F.pad(scores, ((kdim - 1) // 2, (kdim - 1) // 2, qdim - 1, 0), value=0.0)
    else:
        raise ValueError(pad_key)
    return F.conv2d(padded, kernel, padding=0, groups=n_heads // head_sz)


def depthwise_conv(x: torch.Tensor, weight: torch.Tensor, causal: bool = False) -> torch.Tensor:
    """The standalone conv op: out[n,c,p,q] = sum_ij w[c,i,j] x~[n,c,p+i-(R-1), q+j-(S-1)//2].

    Follows convolution_2d_trit.py:418-432 (``pytorch_conv``) for the arithmetic and
    convolution_2d_trit.py:77-78, 108-110, 128-133, 310-313 for the causal rules the
    kernel adds: taps with col>row read as 0, outputs with q>p are +0.  ``weight`` is
    (C,R,S) or (C,1,R,S).  For an even key size the left pad is (S-1)//2 and the
    right pad S-1-(S-1)//2, which is what the kernel's index arithmetic does
    (convolution_2d_trit.py:96-97, 311); the reference's torch restatement only
    covers odd S.
    """
    if weight.dim() == 3:
        weight = weight.unsqueeze(1)
    qdim, kdim = weight.shape[-2], weight.shape[-1]
    if causal:
        x = torch.tril(x)
    left = (kdim - 1) // 2
    padded = F.pad(x, (left, kdim - 1 - left, qdim - 1, 0), value=0.0)
    out = F.conv2d(padded, weight.to(x.dtype), padding=0, groups=x.shape[1])
    if causal:
        out = torch.tril(out)  # exact: multiplies by 1 or replaces by +0
        out = out + 0.0        # canonicalise any -0 left by tril on negative inputs
    return out


# ---------------------------------------------------------------------------
# stage: head mixing
# ---------------------------------------------------------------------------
def head_linear(x: torch.Tensor, weight: torch.Tensor, causal: bool = True,
                output_value: float = 0.0) -> torch.Tensor:
    """y[n,o,p,q] = sum_i W[o,i] x[n,i,p,q]; with ``causal`` every q>p holds ``output_value``.

    Arithmetic follows the transposed nn.Linear of mta_attention_pytorch.py:68,76;
    fill and causal rules follow triton_linear_head.py:294-297 (pre-filled output),
    :111-113 (rows above the block skipped) and :135-139 (diagonal store mask).
    """
    y = F.linear(x.transpose(1, -1), weight.to(x.dtype)).transpose(1, -1).contiguous()
    if causal:
        p, q = x.shape[-2], x.shape[-1]
        upper = torch.triu(torch.ones(p, q, dtype=torch.bool, device=x.device), diagonal=1)
        y = y.masked_fill(upper, output_value)
    return y


# ---------------------------------------------------------------------------
# backward of the two operators: torch.autograd through the forward restatements above
# ---------------------------------------------------------------------------
def depthwise_conv_grads(x, weight, causal, dy):
    """(dx, dw) of ``depthwise_conv`` for the output gradient ``dy``, by torch.autograd.

    What Conv2dTritonFunction.backward computes (convolution_2d_trit.py:336-378).  Pinned in
    tests/test_oracle.py by torch.autograd.gradcheck in fp64 (finite differences), by the C
    restatement of the reference's two backward kernels, and by the adjoint identities
    <conv(x), dy> = <x, dx> = <w, dw>."""
    x = x.detach().clone().requires_grad_(True)
    w = weight.detach().clone().requires_grad_(True)
    y = depthwise_conv(x, w, causal)
    dx, dw = torch.autograd.grad(y, (x, w), dy)
    return dx, dw


def head_linear_grads(x, weight, causal, output_value, dy):
    """(dx, dw) of ``head_linear``, by torch.autograd; what TritonLinearHeadFunction.backward computes
    (triton_linear_head.py:322-370).  Pinned like ``depthwise_conv_grads``."""
    x = x.detach().clone().requires_grad_(True)
    w = weight.detach().clone().requires_grad_(True)
    y = head_linear(x, w, causal, output_value)
    dx, dw = torch.autograd.grad(y, (x, w), dy)
    return dx, dw


# ---------------------------------------------------------------------------
# whole MTA forward
# ---------------------------------------------------------------------------
def mta_forward(xq, xk, xv, mta_kernel, wpsm, mta_kernel_after_sm, wposm, mask=None,
                pad_key: str = "both", dropout: float = 0.0, training: bool = False,
                return_stages: bool = False):
    """Multi-Token Attention forward; (B,H,S,D) x3 -> (B,S,H,D).

    Follows mta_attention_pytorch.py:58-83 line by line.  ``mta_kernel`` and
    ``mta_kernel_after_sm`` are (H,1,R,S); ``wpsm`` and ``wposm`` are the (H,H)
    nn.Linear weights.  The reference builds its scale scalar on "cuda" (:63-65); a
    0-dim tensor on the inputs' device gives the same product, in the inputs' dtype.
    """
    bsz, n_heads = xq.size(0), xq.size(1)
    mask = update_mask(mask, bsz, n_heads, xq, xk.size(-2))
    head_dim = xq.size(-1)
    scale = torch.rsqrt(torch.tensor(head_dim, requires_grad=False, device=xq.device))
    s0 = torch.matmul(xq, xk.transpose(2, 3)) * scale
    s1 = mta_convolution(s0, mask, mta_kernel, pad_key)
    s2 = F.linear(s1.transpose(1, -1), wpsm).transpose(1, -1)
    s3 = s2 + mask
    p0 = F.softmax(s3.float(), dim=-1).type_as(xq)
    p1 = mta_convolution(p0, mask, mta_kernel_after_sm, pad_key)
    p1 = torch.where(mask == NEG_INF, 0.0, p1)
    p2 = F.linear(p1.transpose(1, -1), wposm).transpose(1, -1)
    p2 = F.dropout(p2, p=dropout, training=training)
    out = torch.matmul(p2, xv).transpose(1, 2)
    if return_stages:
        return out, {"s0": s0, "s1": s1, "s2": s2, "p0": p0, "p1": p1, "p2": p2}
    return out


def mta_forward_rows(xq, xk, xv, mta_kernel, wpsm, mta_kernel_after_sm, wposm, row0: int, row1: int):
    """Query rows [row0,row1) of the causal ``mta_forward`` (mask=None, pad_key="both", no dropout)
    without the full S x S tensors; returns (B, row1-row0, H, D).

    A query row of the result depends on the R2-1 probability rows above it (top halo of the
    second conv), each of which depends on the R1-1 score rows above it (top halo of the
    first), on all heads at its own positions and on every key and value.  So the same
    library calls as in ``mta_forward`` are applied to rows [lo,row1) with
    lo = max(0, row0-(R1-1)-(R2-1)) as if row lo were the first row; rows whose halo was
    cut off are wrong and are dropped (none when lo = 0).  Equality with the full form is
    checked in tests/test_oracle.py.
    """
    r1, r2 = mta_kernel.shape[-2], mta_kernel_after_sm.shape[-2]
    sk = xk.size(-2)
    lo = max(0, row0 - (r1 - 1) - (r2 - 1))
    rows = torch.arange(lo, row1, device=xq.device)[:, None]
    cols = torch.arange(sk, device=xq.device)[None, :]
    mask = torch.zeros(row1 - lo, sk, device=xq.device).masked_fill(cols > rows, NEG_INF).type_as(xq)
    mask = mask.repeat(xq.size(0), xq.size(1), 1, 1)
    head_dim = xq.size(-1)
    scale = torch.rsqrt(torch.tensor(head_dim, requires_grad=False, device=xq.device))
    s0 = torch.matmul(xq[:, :, lo:row1], xk.transpose(2, 3)) * scale
    s1 = mta_convolution(s0, mask, mta_kernel, "both")
    s2 = F.linear(s1.transpose(1, -1), wpsm).transpose(1, -1)
    s3 = s2 + mask
    p0 = F.softmax(s3.float(), dim=-1).type_as(xq)
    p1 = mta_convolution(p0, mask, mta_kernel_after_sm, "both")
    p1 = torch.where(mask == NEG_INF, 0.0, p1)
    p2 = F.linear(p1.transpose(1, -1), wposm).transpose(1, -1)
    out = torch.matmul(p2, xv).transpose(1, 2)
    return out[:, row0 - lo:]


# ---------------------------------------------------------------------------
# fused conv-attention forward
# ---------------------------------------------------------------------------
def conv_attention_forward(Q, K, V, conv_weight, causal: bool = True,
                           softmax_scale: Optional[float] = None) -> torch.Tensor:
    """O = softmax(mask(conv(mask0(Q K^T))) * scale) V ; (B,H,S,D) -> (B,H,S,D).

    Follows conv_attention_pytorch.py:33-92: scores are NOT scaled before the conv,
    above-diagonal scores are zeroed before it and set to -inf after it, the scale is
    applied to the conv output, softmax runs in the input dtype.  ``conv_weight`` is
    (H,R,S).
    """
    b, h, s, d = Q.shape
    if softmax_scale is None:
        softmax_scale = 1.0 / (d ** 0.5)
    scores = torch.matmul(Q, K.transpose(-2, -1))
    upper = torch.triu(torch.ones(s, s, device=Q.device), diagonal=1).bool()
    if causal:
        scores = scores.masked_fill(upper, 0)
    r, sk = conv_weight.shape[-2], conv_weight.shape[-1]
    pad_k = (sk - 1) // 2
    # reference: (pad_k, pad_k), key size odd.  For an even key size the right pad is
    # sk-1-pad_k, the index arithmetic of qk_conv_kernel.py:126-129 (pad_k on the left).
    padded = F.pad(scores, (pad_k, sk - 1 - pad_k, r - 1, 0), value=0.0)
    conv = F.conv2d(padded, conv_weight.to(Q.dtype).unsqueeze(1), padding=0, groups=h)
    if causal:
        conv = conv.masked_fill(upper, NEG_INF)
    attn = F.softmax(conv * softmax_scale, dim=-1)
    return torch.matmul(attn, V)


def conv_attention_scores(Q, K, conv_weight, causal: bool = True, softmax_scale: Optional[float] = None):
    """The logits ``conv_attention_forward`` feeds its softmax: mask(conv(mask0(Q K^T))) * scale, (B,H,S,S);
    conv_attention_pytorch.py:44-66.  Its row-wise ``torch.logsumexp`` is the statistic the reference's fused
    kernel calls M (conv_attention_triton.py:352-355).  Pinned in tests/test_oracle.py by
    softmax(scores) V == conv_attention_forward and exp(scores - lse) rows summing to 1."""
    b, h, s, d = Q.shape
    if softmax_scale is None:
        softmax_scale = 1.0 / (d ** 0.5)
    scores = torch.matmul(Q, K.transpose(-2, -1))
    upper = torch.triu(torch.ones(s, s, device=Q.device), diagonal=1).bool()
    if causal:
        scores = scores.masked_fill(upper, 0)
    r, sk = conv_weight.shape[-2], conv_weight.shape[-1]
    pad_k = (sk - 1) // 2
    padded = F.pad(scores, (pad_k, sk - 1 - pad_k, r - 1, 0), value=0.0)
    conv = F.conv2d(padded, conv_weight.to(Q.dtype).unsqueeze(1), padding=0, groups=h)
    if causal:
        conv = conv.masked_fill(upper, NEG_INF)
    return conv * softmax_scale


def conv_attention_rows(Q, K, V, conv_weight, row0: int, row1: int, causal: bool = True,
                        softmax_scale: Optional[float] = None) -> torch.Tensor:
    """Rows [row0,row1) of ``conv_attention_forward`` without the full S x S tensor.

    Query rows are independent given all keys and values plus the R-1 query rows
    above them (the conv's top halo), so the same library calls are applied to the
    slab rows [row0-(R-1), row1) and the halo rows are dropped afterwards.  Equality
    with the full form is checked in tests/test_oracle.py.
    """
    b, h, s, d = Q.shape
    if softmax_scale is None:
        softmax_scale = 1.0 / (d ** 0.5)
    r, sk = conv_weight.shape[-2], conv_weight.shape[-1]
    lo = max(0, row0 - (r - 1))
    top_pad = (r - 1) - (row0 - lo)
    scores = torch.matmul(Q[:, :, lo:row1], K.transpose(-2, -1))
    rows = torch.arange(lo, row1, device=Q.device)[:, None]
    cols = torch.arange(s, device=Q.device)[None, :]
    upper = cols > rows
    if causal:
        scores = scores.masked_fill(upper, 0)
    pad_k = (sk - 1) // 2
    padded = F.pad(scores, (pad_k, sk - 1 - pad_k, top_pad, 0), value=0.0)
    conv = F.conv2d(padded, conv_weight.to(Q.dtype).unsqueeze(1), padding=0, groups=h)
    if causal:
        conv = conv.masked_fill(upper[row0 - lo:], NEG_INF)
    attn = F.softmax(conv * softmax_scale, dim=-1)
    return torch.matmul(attn, V)


# ---------------------------------------------------------------------------
# parameter conventions and seeded inputs shared by tests, smoke and bench
# ---------------------------------------------------------------------------
def identity_conv_kernel(n_heads: int, r: int, s: int, dtype=torch.float32) -> torch.Tensor:
    """(H,R,S) kernel that passes scores through: 1.0 at [R-1, S//2].

    mta_attention_pytorch.py:166-190 and conv_attention_pytorch.py:25-31.
    """
    w = torch.zeros(n_heads, r, s, dtype=dtype)
    w[:, -1, s // 2] = 1.0
    return w


def block_diag_head_weight(n_heads: int, group: int, std: float, gen: torch.Generator,
                           dtype=torch.float32) -> torch.Tensor:
    """(H,H) head-mix weight: I + N(0,std) inside group x group diagonal blocks, 0 elsewhere."""
    w = torch.zeros(n_heads, n_heads)
    for g in range(0, n_heads, group):
        w[g:g + group, g:g + group] = torch.eye(group) + std * torch.randn(group, group, generator=gen)
    return w.to(dtype)


def seeded_qkv(b, h, s, d, dtype, seed=123):
    """q,k,v ~ N(0,1) drawn in fp32 from a CPU generator and cast (seed of compare_mta_attention.py:71)."""
    g = torch.Generator().manual_seed(seed)
    return tuple(torch.randn(b, h, s, d, generator=g).to(dtype) for _ in range(3))


def seeded_conv_weight(h, r, s, std, dtype, seed=124, identity_tap=True):
    g = torch.Generator().manual_seed(seed)
    w = std * torch.randn(h, r, s, generator=g)
    if identity_tap:
        w[:, r - 1, s // 2] += 1.0
    return w.to(dtype)


def tolerance(dtype):
    """Parity bars: fp32 rtol 1e-4 (atol 1e-5 for entries near 0); bf16/fp16 atol 2e-2."""
    if dtype == torch.float32:
        return dict(rtol=1e-4, atol=1e-5)
    return dict(rtol=1.6e-2, atol=2e-2)


__all__ = [n for n in dir() if not n.startswith("_")]
_ = math
