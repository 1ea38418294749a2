"""Tensor-level wrappers over the C ABI: torch supplies device memory and the stream,
every computation happens in libmta_hip.so.  No fallback: a CPU tensor or a missing
library raises.
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from . import _lib

_DTYPE_CODE = {torch.float32: _lib.MTA_F32, torch.bfloat16: _lib.MTA_BF16, torch.float16: _lib.MTA_F16}


def _code(t: torch.Tensor, what: str) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise TypeError(f"{what}: dtype {t.dtype} is not supported (float32, bfloat16, float16)") from None


def _device_tensor(t: torch.Tensor, what: str) -> torch.Tensor:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{what} must be a torch.Tensor")
    if not t.is_cuda:
        raise RuntimeError(f"{what} lives on {t.device}: the MTA kernels only run on an AMD GPU "
                           "(there is no CPU path)")
    return t if t.is_contiguous() else t.contiguous()


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _causal_mode(causal: bool, fill_upper: bool) -> int:
    """The `causal` argument of the conv / head-mixing entry points: 0, 1, or MTA_CAUSAL_LOWER_ONLY."""
    if not causal:
        return 0
    return 1 if fill_upper else _lib.MTA_CAUSAL_LOWER_ONLY


def _out_like(x: torch.Tensor, out: Optional[torch.Tensor]) -> torch.Tensor:
    if out is None:
        return torch.empty_like(x, memory_format=torch.contiguous_format)
    if out.shape != x.shape or out.dtype != x.dtype or out.device != x.device or not out.is_contiguous():
        raise ValueError("out must be a contiguous tensor with the input's shape, dtype and device")
    return out


def conv2d_causal(x: torch.Tensor, weight: torch.Tensor, causal: bool, in_scale: Optional[float] = None,
                  out: Optional[torch.Tensor] = None, fill_upper: bool = True) -> torch.Tensor:
    """Depthwise conv over (N,C,H,W) with a (C,R,S) kernel; see mta_conv2d_fwd in include/mta_hip.h.

    ``fill_upper=False`` (causal, no ``in_scale``): for a consumer that never reads above the diagonal; what lies
    there is unspecified (mta_conv2d_tril_fwd)."""
    x = _device_tensor(x, "input")
    weight = _device_tensor(weight.detach(), "weight")
    if x.dim() != 4 or weight.dim() != 3:
        raise ValueError(f"expected input (N,C,H,W) and weight (C,R,S), got {tuple(x.shape)} and {tuple(weight.shape)}")
    n, c, h, w = x.shape
    c_out, r, s = weight.shape
    # same check and message as convolution_2d_trit.py:306
    assert c == c_out, "This implementation assumes depthwise convolution (C_in == C_out)"
    y = _out_like(x, out)
    lib = _lib.load()
    with torch.cuda.device(x.device):
        if in_scale is None and causal and not fill_upper:
            rc = lib.mta_conv2d_tril_fwd(x.data_ptr(), weight.data_ptr(), y.data_ptr(), n, c, h, w, r, s,
                                         _code(x, "input"), _code(weight, "weight"), _stream(x))
        elif in_scale is None:
            rc = lib.mta_conv2d_fwd(x.data_ptr(), weight.data_ptr(), y.data_ptr(), n, c, h, w, r, s, int(bool(causal)),
                                    _code(x, "input"), _code(weight, "weight"), _stream(x))
        else:
            rc = lib.mta_conv2d_scaled_fwd(x.data_ptr(), weight.data_ptr(), y.data_ptr(), n, c, h, w, r, s,
                                           _causal_mode(causal, fill_upper), float(in_scale), _code(x, "input"),
                                           _code(weight, "weight"), _stream(x))
    _lib.check(rc, "mta_conv2d_fwd")
    return y


def headmix(x: torch.Tensor, weight: torch.Tensor, causal: bool = True, fill: float = 0.0,
            group_size: Optional[int] = None, out: Optional[torch.Tensor] = None, fill_upper: bool = True) -> torch.Tensor:
    """y[n,o,p,q] = sum_i W[o,i] x[n,i,p,q]; see mta_headmix_fwd in include/mta_hip.h.

    ``fill_upper=False`` (causal): for a consumer that never reads above the diagonal; vectors wholly above it are not
    written (mta_headmix_tril_fwd)."""
    x = _device_tensor(x, "input")
    weight = _device_tensor(weight.detach(), "weight")
    if x.dim() != 4:
        raise ValueError(f"expected input (N,C,P,Q), got {tuple(x.shape)}")
    n, c, p, q = x.shape
    l = weight.shape[0]
    # same checks and messages as triton_linear_head.py:286-290
    assert tuple(weight.shape) == (l, l), f"Weight must be square matrix, got {weight.shape}"
    assert c == l, f"Channel dimension {c} must match weight dimension {l}"
    y = _out_like(x, out)
    with torch.cuda.device(x.device):
        if causal and not fill_upper:
            rc = _lib.load().mta_headmix_tril_fwd(x.data_ptr(), weight.data_ptr(), y.data_ptr(), n, c, p, q,
                                                  int(group_size or 0), _code(x, "input"), _code(weight, "weight"),
                                                  _stream(x))
        else:
            rc = _lib.load().mta_headmix_fwd(x.data_ptr(), weight.data_ptr(), y.data_ptr(), n, c, p, q,
                                             int(group_size or 0), int(bool(causal)), float(fill), _code(x, "input"),
                                             _code(weight, "weight"), _stream(x))
    _lib.check(rc, "mta_headmix_fwd")
    return y


def _workspace(nbytes: int, device) -> torch.Tensor:
    return torch.empty(max(int(nbytes), 16), dtype=torch.uint8, device=device)


def conv2d_bwd_input(dy: torch.Tensor, weight: torch.Tensor, causal: bool, fill_upper: bool = True,
                     out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Gradient of ``conv2d_causal`` with respect to its input; see mta_conv2d_bwd_input.  ``fill_upper=False``
    (causal): for a consumer that never reads above the diagonal."""
    dy = _device_tensor(dy, "grad_output")
    weight = _device_tensor(weight.detach(), "weight")
    n, c, h, w = dy.shape
    c_out, r, s = weight.shape
    assert c == c_out, "This implementation assumes depthwise convolution (C_in == C_out)"
    dx = _out_like(dy, out)
    with torch.cuda.device(dy.device):
        rc = _lib.load().mta_conv2d_bwd_input(dy.data_ptr(), weight.data_ptr(), dx.data_ptr(), n, c, h, w, r, s,
                                              _causal_mode(causal, fill_upper), _code(dy, "grad_output"), _code(weight, "weight"),
                                              _stream(dy))
    _lib.check(rc, "mta_conv2d_bwd_input")
    return dx


def conv2d_bwd_weight(x: torch.Tensor, dy: torch.Tensor, kernel_size, causal: bool) -> torch.Tensor:
    """Gradient of ``conv2d_causal`` with respect to its (C,R,S) kernel, in fp32; see mta_conv2d_bwd_weight."""
    x = _device_tensor(x, "input")
    dy = _device_tensor(dy, "grad_output")
    if x.shape != dy.shape or x.dtype != dy.dtype:
        raise ValueError("input and grad_output must share shape and dtype")
    n, c, h, w = x.shape
    r, s = kernel_size
    lib = _lib.load()
    dw = torch.empty((c, r, s), dtype=torch.float32, device=x.device)
    nbytes = lib.mta_conv2d_bwd_weight_workspace(n, c, h, w, r, s)
    ws = _workspace(nbytes, x.device)
    with torch.cuda.device(x.device):
        rc = lib.mta_conv2d_bwd_weight(x.data_ptr(), dy.data_ptr(), dw.data_ptr(), ws.data_ptr(), ws.numel(), n, c, h, w,
                                       r, s, int(bool(causal)), _code(x, "input"), _stream(x))
    _lib.check(rc, "mta_conv2d_bwd_weight")
    return dw


def headmix_bwd_input(dy: torch.Tensor, weight: torch.Tensor, causal: bool = True,
                      group_size: Optional[int] = None, fill_upper: bool = True,
                      out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Gradient of ``headmix`` with respect to its input (+0 above the diagonal); see mta_headmix_bwd_input.
    ``fill_upper=False`` (causal): for a consumer that never reads above the diagonal."""
    dy = _device_tensor(dy, "grad_output")
    weight = _device_tensor(weight.detach(), "weight")
    n, c, p, q = dy.shape
    assert tuple(weight.shape) == (c, c), f"Weight must be ({c},{c}), got {tuple(weight.shape)}"
    dx = _out_like(dy, out)
    with torch.cuda.device(dy.device):
        rc = _lib.load().mta_headmix_bwd_input(dy.data_ptr(), weight.data_ptr(), dx.data_ptr(), n, c, p, q,
                                               int(group_size or 0), _causal_mode(causal, fill_upper), _code(dy, "grad_output"),
                                               _code(weight, "weight"), _stream(dy))
    _lib.check(rc, "mta_headmix_bwd_input")
    return dx


def headmix_bwd_weight(x: torch.Tensor, dy: torch.Tensor, causal: bool = True) -> torch.Tensor:
    """Gradient of ``headmix`` with respect to its (C,C) weight, dense, in fp32; see mta_headmix_bwd_weight."""
    x = _device_tensor(x, "input")
    dy = _device_tensor(dy, "grad_output")
    if x.shape != dy.shape or x.dtype != dy.dtype:
        raise ValueError("input and grad_output must share shape and dtype")
    n, c, p, q = x.shape
    lib = _lib.load()
    dw = torch.empty((c, c), dtype=torch.float32, device=x.device)
    nbytes = lib.mta_headmix_bwd_weight_workspace(n, c, p, q)
    if nbytes <= 0:
        raise ValueError(f"mta_headmix_bwd_weight: no kernel for {c} heads (at most 128)")
    ws = _workspace(nbytes, x.device)
    with torch.cuda.device(x.device):
        rc = lib.mta_headmix_bwd_weight(x.data_ptr(), dy.data_ptr(), dw.data_ptr(), ws.data_ptr(), ws.numel(), n, c, p, q,
                                        int(bool(causal)), _code(x, "input"), _stream(x))
    _lib.check(rc, "mta_headmix_bwd_weight")
    return dw


def headmix_softmax(x: torch.Tensor, w1: Optional[torch.Tensor], w2: Optional[torch.Tensor], causal: bool = True,
                    group_size: Optional[int] = None, out: Optional[torch.Tensor] = None,
                    fill_upper: bool = True, key_bias: Optional[torch.Tensor] = None,
                    first_visible: Optional[torch.Tensor] = None) -> torch.Tensor:
    """mix(w1) -> causal row softmax -> mix(w2) in one pass; see mta_headmix_softmax_fwd.

    ``first_visible``: int32 (N,P), the first visible key of every query row (band mask); see
    mta_headmix_softmax_band_fwd.

    ``fill_upper=False`` leaves everything above the diagonal unwritten (for consumers that never read it).
    ``key_bias``: fp32 (N,Q), added to the mixed scores ahead of the softmax (0 = keep, -inf = key hidden); see
    mta_headmix_softmax_bias_fwd."""
    x = _device_tensor(x, "input")
    if x.dim() != 4:
        raise ValueError(f"expected input (N,C,P,Q), got {tuple(x.shape)}")
    n, c, p, q = x.shape
    ws = []
    for w in (w1, w2):
        if w is not None:
            w = _device_tensor(w.detach(), "weight")
            assert tuple(w.shape) == (c, c), f"Weight must be ({c},{c}), got {tuple(w.shape)}"
        ws.append(w)
    present = [w for w in ws if w is not None]
    if len(present) == 2 and present[0].dtype != present[1].dtype:
        raise TypeError("w1 and w2 must share a dtype")
    wcode = _code(present[0], "weight") if present else _lib.MTA_F32
    if key_bias is not None:
        key_bias = _device_tensor(key_bias, "key_bias")
        if key_bias.dtype != torch.float32 or tuple(key_bias.shape) != (n, q):
            raise ValueError(f"key_bias must be fp32 of shape ({n},{q}), got {key_bias.dtype} {tuple(key_bias.shape)}")
    if first_visible is not None:
        first_visible = _device_tensor(first_visible, "first_visible")
        if first_visible.dtype != torch.int32 or tuple(first_visible.shape) != (n, p):
            raise ValueError(f"first_visible must be int32 of shape ({n},{p}), got {first_visible.dtype} "
                             f"{tuple(first_visible.shape)}")
    y = _out_like(x, out)
    with torch.cuda.device(x.device):
        rc = _lib.load().mta_headmix_softmax_band_fwd(
            x.data_ptr(), ws[0].data_ptr() if ws[0] is not None else None,
            ws[1].data_ptr() if ws[1] is not None else None, key_bias.data_ptr() if key_bias is not None else None,
            first_visible.data_ptr() if first_visible is not None else None,
            y.data_ptr(), n, c, p, q, int(group_size or 0), int(bool(causal)), int(bool(fill_upper)), _code(x, "input"),
            wcode, _stream(x))
    _lib.check(rc, "mta_headmix_softmax_band_fwd")
    return y


def softmax_bwd(p: torch.Tensor, dp: torch.Tensor, causal: bool = True, fill_upper: bool = True) -> torch.Tensor:
    """Gradient of the row softmax from its stored output ``p`` (N,C,P,Q) and the incoming gradient ``dp``; see
    mta_softmax_bwd.  ``fill_upper=False`` (causal) leaves the result above the diagonal unwritten."""
    p = _device_tensor(p, "probabilities")
    dp = _device_tensor(dp, "grad_output")
    if p.dim() != 4 or p.shape != dp.shape or p.dtype != dp.dtype:
        raise ValueError("probabilities and grad_output must be (N,C,P,Q) tensors of one shape and dtype")
    n, c, rows, q = p.shape
    dx = torch.empty_like(p, memory_format=torch.contiguous_format)
    with torch.cuda.device(p.device):
        rc = _lib.load().mta_softmax_bwd(p.data_ptr(), dp.data_ptr(), dx.data_ptr(), n, c, rows, q, int(bool(causal)),
                                         int(bool(fill_upper)), _code(p, "probabilities"), _stream(p))
    _lib.check(rc, "mta_softmax_bwd")
    return dx


def conv2d_headmix(x: torch.Tensor, w_conv: torch.Tensor, w_mix: torch.Tensor, causal: bool = True,
                   group_size: Optional[int] = None, out: Optional[torch.Tensor] = None,
                   fill_upper: bool = True) -> Optional[torch.Tensor]:
    """Depthwise causal conv, then head mixing, in one pass; see mta_conv2d_headmix_fwd.  Returns None when the
    library has no kernel for the mixing-group size (the caller then runs the two operators one after the other)."""
    x = _device_tensor(x, "input")
    if x.dim() != 4:
        raise ValueError(f"expected input (N,C,H,W), got {tuple(x.shape)}")
    n, c, h, w = x.shape
    w_conv = _device_tensor(w_conv.detach(), "conv weight")
    w_mix = _device_tensor(w_mix.detach(), "mix weight")
    assert w_conv.dim() == 3 and w_conv.size(0) == c, "Input and weight channels must match"
    assert tuple(w_mix.shape) == (c, c), f"Weight must be ({c},{c}), got {tuple(w_mix.shape)}"
    y = _out_like(x, out)
    with torch.cuda.device(x.device):
        rc = _lib.load().mta_conv2d_headmix_fwd(
            x.data_ptr(), w_conv.data_ptr(), w_mix.data_ptr(), y.data_ptr(), n, c, h, w, w_conv.size(1), w_conv.size(2),
            int(group_size or 0), int(bool(causal)), int(bool(fill_upper)), _code(x, "input"), _code(w_conv, "weight"),
            _code(w_mix, "weight"), _stream(x))
    if rc == _lib.MTA_ERR_UNSUPPORTED:
        return None
    _lib.check(rc, "mta_conv2d_headmix_fwd")
    return y


def conv_attn_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, weight: torch.Tensor, causal: bool,
                  softmax_scale: Optional[float] = None, out: Optional[torch.Tensor] = None,
                  return_lse: bool = False):
    """O = softmax(mask(conv(mask0(QK^T))) * scale) V for (B,H,S,D) inputs; see mta_conv_attn_fwd.

    With ``return_lse`` the result is (O, lse), lse (B,H,S) fp32 = log-sum-exp of each row's scaled conv scores."""
    q = _device_tensor(q, "Q")
    k = _device_tensor(k, "K")
    v = _device_tensor(v, "V")
    weight = _device_tensor(weight.detach(), "W")
    if q.dim() != 4 or q.shape != k.shape or q.shape != v.shape:
        raise ValueError(f"Q, K, V must share a (B,H,S,D) shape, got {tuple(q.shape)}, {tuple(k.shape)}, {tuple(v.shape)}")
    if not (q.dtype == k.dtype == v.dtype):
        raise TypeError("Q, K, V must share a dtype")
    b, h, s, d = q.shape
    # same check as conv_attention_triton.py:369
    assert weight.dim() == 3 and weight.shape[0] == h, "CHANNEL_DIM == NUM_HEADS"
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(d)
    o = _out_like(q, out)
    lse = torch.empty((b, h, s), dtype=torch.float32, device=q.device) if return_lse else None
    with torch.cuda.device(q.device):
        rc = _lib.load().mta_conv_attn_fwd_lse(q.data_ptr(), k.data_ptr(), v.data_ptr(), weight.data_ptr(), o.data_ptr(),
                                               lse.data_ptr() if return_lse else None, b, h, s, d, weight.shape[1],
                                               weight.shape[2], int(bool(causal)), float(softmax_scale), _code(q, "Q"),
                                               _code(weight, "W"), _stream(q))
    _lib.check(rc, "mta_conv_attn_fwd")
    return (o, lse) if return_lse else o


def qk_conv(q: torch.Tensor, k: torch.Tensor, weight: torch.Tensor, causal: bool, scale: float,
            fill_upper: bool = True, out: Optional[torch.Tensor] = None,
            first_visible: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """scale * conv(mask0(Q K^T)) as a (B,H,S,S) tensor without materialising Q K^T; see mta_qk_conv_fwd.

    ``first_visible``: int32 (B,S), band mask (requires ``causal``): key k of row p counts only when
    first_visible[b,p] <= k <= p; see mta_qk_conv_band_fwd.

    Returns ``None`` when the library has no kernel for this dtype / size combination (the caller then
    takes matmul + conv2d_causal).  With ``fill_upper=False`` entries above the diagonal are left unwritten."""
    q = _device_tensor(q, "Q")
    k = _device_tensor(k, "K")
    weight = _device_tensor(weight.detach(), "W")
    if q.dim() != 4 or q.shape != k.shape or q.dtype != k.dtype:
        raise ValueError(f"Q and K must share a (B,H,S,D) shape and dtype, got {tuple(q.shape)}, {tuple(k.shape)}")
    b, h, s, d = q.shape
    assert weight.dim() == 3 and weight.shape[0] == h, "conv weight must be (H,R,S)"
    if out is None:
        out = torch.empty((b, h, s, s), dtype=q.dtype, device=q.device)
    elif out.shape != (b, h, s, s) or out.dtype != q.dtype or out.device != q.device or not out.is_contiguous():
        raise ValueError("out must be a contiguous (B,H,S,S) tensor of the inputs' dtype and device")
    if first_visible is not None:
        if not causal:
            raise ValueError("a band mask implies the causal rule")
        first_visible = _device_tensor(first_visible, "first_visible")
        if first_visible.dtype != torch.int32 or tuple(first_visible.shape) != (b, s):
            raise ValueError(f"first_visible must be int32 of shape ({b},{s}), got {first_visible.dtype} "
                             f"{tuple(first_visible.shape)}")
    with torch.cuda.device(q.device):
        if first_visible is not None:
            rc = _lib.load().mta_qk_conv_band_fwd(q.data_ptr(), k.data_ptr(), weight.data_ptr(), first_visible.data_ptr(),
                                                  out.data_ptr(), b, h, s, d, weight.shape[1], weight.shape[2], float(scale),
                                                  int(bool(fill_upper)), _code(q, "Q"), _code(weight, "W"), _stream(q))
        else:
            rc = _lib.load().mta_qk_conv_fwd(q.data_ptr(), k.data_ptr(), weight.data_ptr(), out.data_ptr(), b, h, s, d,
                                             weight.shape[1], weight.shape[2], int(bool(causal)), float(scale),
                                             int(bool(fill_upper)), _code(q, "Q"), _code(weight, "W"), _stream(q))
    if rc in (_lib.MTA_ERR_UNSUPPORTED, -7):
        return None
    _lib.check(rc, "mta_qk_conv_fwd")
    return out


def qk_conv_supported(q: torch.Tensor, k: torch.Tensor, weight: torch.Tensor) -> bool:
    """Whether ``qk_conv`` has a kernel for these tensors (a host-side question to the library: nothing is launched)."""
    if q.dim() != 4 or q.shape != k.shape or q.dtype != k.dtype or weight.dim() != 3:
        return False
    if q.dtype not in _DTYPE_CODE or weight.dtype not in _DTYPE_CODE:
        return False
    return bool(_lib.load().mta_qk_conv_supported(q.size(2), q.size(3), weight.size(1), weight.size(2),
                                                  _DTYPE_CODE[q.dtype], _DTYPE_CODE[weight.dtype]))


def causal_pv(p: torch.Tensor, v: torch.Tensor, causal: bool,
              first_visible: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """P V for P (B,H,S,S), V (B,H,S,D), reading only the lower triangle of P when causal; see mta_causal_pv_fwd.

    ``first_visible``: int32 (B,S), band mask (P is 0 ahead of a row's first visible key): the key blocks no row of a
    query block sees are not read; see mta_causal_pv_band_fwd.
    Returns ``None`` when unsupported (the caller then uses torch.matmul on a fully defined P)."""
    p = _device_tensor(p, "P")
    v = _device_tensor(v, "V")
    if p.dim() != 4 or v.dim() != 4 or p.shape[:3] != v.shape[:3] or p.shape[2] != p.shape[3] or p.dtype != v.dtype:
        return None
    b, h, s, d = v.shape
    out = torch.empty_like(v)
    if first_visible is not None:
        first_visible = _device_tensor(first_visible, "first_visible")
        if first_visible.dtype != torch.int32 or tuple(first_visible.shape) != (b, s):
            raise ValueError(f"first_visible must be int32 of shape ({b},{s}), got {first_visible.dtype} "
                             f"{tuple(first_visible.shape)}")
    with torch.cuda.device(p.device):
        rc = _lib.load().mta_causal_pv_band_fwd(p.data_ptr(), v.data_ptr(),
                                                first_visible.data_ptr() if first_visible is not None else None,
                                                out.data_ptr(), b, h, s, d, int(bool(causal)), _code(p, "P"), _stream(p))
    if rc in (_lib.MTA_ERR_UNSUPPORTED, -7):
        return None
    _lib.check(rc, "mta_causal_pv_fwd")
    return out


# ---------------------------------------------------------------------------------------
# the causal forward's three stages over score tensors in the triangular layout (include/mta_hip.h): what lies on and
# below the diagonal only, rows padded to 64 keys, the heads of a mixing group interleaved by rows
# ---------------------------------------------------------------------------------------
def tri_row_offset(p: int) -> int:
    """Elements of one head ahead of row p in the triangular layout; tri_row_offset(S) is a head's size."""
    a = p >> 6
    return 2048 * a * (a + 1) + (p & 63) * 64 * (a + 1)


def _band_arg(first_visible, b, s):
    if first_visible is None:
        return None
    first_visible = _device_tensor(first_visible, "first_visible")
    if first_visible.dtype != torch.int32 or tuple(first_visible.shape) != (b, s):
        raise ValueError(f"first_visible must be int32 of shape ({b},{s}), got {first_visible.dtype} "
                         f"{tuple(first_visible.shape)}")
    return first_visible


def tri_route_supported(q: torch.Tensor, k: torch.Tensor, conv_weight: torch.Tensor, group: int, w1, w2, band: bool,
                        out_planes: bool = False, key_bias: bool = False) -> bool:
    """Whether the triangular-layout kernels exist for these tensors (host-side questions to the library);
    ``out_planes``: the softmax stage hands on (B,H,S,S) planes (then only the first two kernels are asked for)."""
    if not qk_conv_supported(q, k, conv_weight) or q.dtype not in (torch.bfloat16, torch.float16):
        return False
    b, h, s, d = q.shape
    ws = [w for w in (w1, w2) if w is not None]
    if not ws or any(w.dtype != q.dtype or w.data_ptr() % 4 for w in ws) or h % group != 0:
        return False
    if group * tri_row_offset(s) >= 2 ** 31 or not causal_pv_supported(q.dtype, s, d):
        return False
    return bool(_lib.load().mta_headmix_softmax_tri_supported(h, s, group, int(out_planes), _DTYPE_CODE[q.dtype],
                                                              _DTYPE_CODE[ws[0].dtype], int(w1 is not None),
                                                              int(w2 is not None), int(band), int(key_bias)))


def qk_conv_tri(q: torch.Tensor, k: torch.Tensor, weight: torch.Tensor, scale: float, group: int,
                first_visible: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal scale * conv(mask0(Q K^T)) in the triangular layout with groups of ``group`` heads: a flat tensor of
    B*H*tri_row_offset(S) elements; see mta_qk_conv_tri_fwd."""
    q = _device_tensor(q, "Q")
    k = _device_tensor(k, "K")
    weight = _device_tensor(weight.detach(), "W")
    if q.dim() != 4 or q.shape != k.shape or q.dtype != k.dtype:
        raise ValueError(f"Q and K must share a (B,H,S,D) shape and dtype, got {tuple(q.shape)}, {tuple(k.shape)}")
    b, h, s, d = q.shape
    assert weight.dim() == 3 and weight.shape[0] == h, "conv weight must be (H,R,S)"
    first_visible = _band_arg(first_visible, b, s)
    out = torch.empty((b * h * tri_row_offset(s),), dtype=q.dtype, device=q.device)
    with torch.cuda.device(q.device):
        rc = _lib.load().mta_qk_conv_tri_fwd(q.data_ptr(), k.data_ptr(), weight.data_ptr(),
                                             first_visible.data_ptr() if first_visible is not None else None,
                                             out.data_ptr(), b, h, s, d, weight.shape[1], weight.shape[2], float(scale),
                                             int(group), _code(q, "Q"), _code(weight, "W"), _stream(q))
    _lib.check(rc, "mta_qk_conv_tri_fwd")
    return out


def headmix_softmax_tri(x: torch.Tensor, w1: Optional[torch.Tensor], w2: Optional[torch.Tensor], n: int, c: int, s: int,
                        group: int, first_visible: Optional[torch.Tensor] = None, out_planes: bool = False,
                        key_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """mix(w1) -> causal row softmax -> mix(w2) over a flat tensor in the triangular layout (mixing groups = the layout's
    groups); the result in the same layout or, with ``out_planes``, as an (N,C,S,S) tensor with nothing written above the
    diagonal; see mta_headmix_softmax_tri_fwd."""
    x = _device_tensor(x, "input")
    if x.dim() != 1 or x.numel() != n * c * tri_row_offset(s):
        raise ValueError(f"expected a flat tensor of {n * c * tri_row_offset(s)} elements, got {tuple(x.shape)}")
    ws = []
    for w in (w1, w2):
        if w is not None:
            w = _device_tensor(w.detach(), "weight")
            assert tuple(w.shape) == (c, c), f"Weight must be ({c},{c}), got {tuple(w.shape)}"
        ws.append(w)
    present = [w for w in ws if w is not None]
    if not present or any(w.dtype != present[0].dtype for w in present):
        raise TypeError("one or two weights of one dtype")
    first_visible = _band_arg(first_visible, n, s)
    if key_bias is not None:
        key_bias = _device_tensor(key_bias, "key_bias")
        if key_bias.dtype != torch.float32 or tuple(key_bias.shape) != (n, s) or not key_bias.is_contiguous():
            raise ValueError(f"key_bias must be a contiguous fp32 tensor of shape ({n},{s})")
    y = torch.empty((n, c, s, s), dtype=x.dtype, device=x.device) if out_planes else torch.empty_like(x)
    with torch.cuda.device(x.device):
        rc = _lib.load().mta_headmix_softmax_tri_fwd(
            x.data_ptr(), ws[0].data_ptr() if ws[0] is not None else None, ws[1].data_ptr() if ws[1] is not None else None,
            key_bias.data_ptr() if key_bias is not None else None,
            first_visible.data_ptr() if first_visible is not None else None, y.data_ptr(), n, c, s, int(group),
            int(bool(out_planes)), _code(x, "input"), _code(present[0], "weight"), _stream(x))
    _lib.check(rc, "mta_headmix_softmax_tri_fwd")
    return y


def causal_pv_tri(p: torch.Tensor, v: torch.Tensor, group: int, first_visible: Optional[torch.Tensor] = None) -> torch.Tensor:
    """P V with P a flat tensor in the triangular layout and V (B,H,S,D); see mta_causal_pv_tri_fwd."""
    p = _device_tensor(p, "P")
    v = _device_tensor(v, "V")
    b, h, s, d = v.shape
    if p.dim() != 1 or p.numel() != b * h * tri_row_offset(s) or p.dtype != v.dtype:
        raise ValueError(f"expected a flat tensor of {b * h * tri_row_offset(s)} elements of V's dtype")
    first_visible = _band_arg(first_visible, b, s)
    out = torch.empty_like(v)
    with torch.cuda.device(p.device):
        rc = _lib.load().mta_causal_pv_tri_fwd(p.data_ptr(), v.data_ptr(),
                                               first_visible.data_ptr() if first_visible is not None else None,
                                               out.data_ptr(), b, h, s, d, int(group), _code(p, "P"), _stream(p))
    _lib.check(rc, "mta_causal_pv_tri_fwd")
    return out


def _tri_index(b: int, h: int, s: int, group: int, device) -> torch.Tensor:
    """Flat positions of the elements (b, h, p, q <= p) of the triangular layout, as a (B,H,S,S) int64 tensor (-1 above the
    diagonal)."""
    rows = torch.arange(s, device=device)
    a = rows >> 6
    off = 2048 * a * (a + 1) + (rows & 63) * 64 * (a + 1)            # (S,)
    length = (a + 1) * 64
    bh = torch.arange(b * h, device=device)
    gbase = (bh // group) * (group * tri_row_offset(s))              # (B*H,)
    idx = (gbase[:, None, None] + (group * off)[None, :, None] + ((bh % group)[:, None, None] * length[None, :, None])
           + rows[None, None, :])
    idx = idx.masked_fill(rows[None, None, :] > rows[None, :, None], -1)
    return idx.view(b, h, s, s)


def tri_unpack(x: torch.Tensor, b: int, h: int, s: int, group: int) -> torch.Tensor:
    """(B,H,S,S) tensor (zero above the diagonal) from a flat tensor in the triangular layout; for tests and inspection."""
    idx = _tri_index(b, h, s, group, x.device)
    out = x[idx.clamp_min(0)]
    return out.masked_fill(idx < 0, 0)


def tri_pack(x: torch.Tensor, group: int, pad_value: float = float("nan")) -> torch.Tensor:
    """The inverse of tri_unpack (padding and nothing else filled with ``pad_value``); for tests and inspection."""
    b, h, s, _ = x.shape
    idx = _tri_index(b, h, s, group, x.device)
    out = torch.full((b * h * tri_row_offset(s),), pad_value, dtype=x.dtype, device=x.device)
    keep = idx >= 0
    out[idx[keep]] = x[keep]
    return out


def band_zero_(x: torch.Tensor, first_visible: torch.Tensor) -> Optional[torch.Tensor]:
    """In place: x[n,c,p,q] = 0 for q < first_visible[n,p] (what the reference's ``torch.where(mask == -inf, 0, scores)``
    behind the post-softmax conv does under a band mask); see mta_band_zero_fwd.  Returns ``None`` when unsupported."""
    x = _device_tensor(x, "input")
    if x.dim() != 4 or x.shape[2] != x.shape[3] or not x.is_contiguous():
        raise ValueError(f"expected a contiguous (N,C,S,S) tensor, got {tuple(x.shape)}")
    n, c, s, _ = x.shape
    first_visible = _band_arg(first_visible, n, s)
    with torch.cuda.device(x.device):
        rc = _lib.load().mta_band_zero_fwd(x.data_ptr(), first_visible.data_ptr(), n, c, s, _code(x, "input"), _stream(x))
    if rc == _lib.MTA_ERR_UNSUPPORTED:
        return None
    _lib.check(rc, "mta_band_zero_fwd")
    return x


def mask_fill(x: torch.Tensor, visible: torch.Tensor, neg_inf: bool, causal: bool,
              out: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """``visible ? x : (-inf if neg_inf else 0)`` for a mask tensor of arbitrary content: ``visible`` is uint8 (or bool),
    non-zero = attend, of shape (1|N, 1|C, P, Q); with ``causal`` only keys q <= p are read and written.  ``out`` may be
    ``x`` (in place).  See mta_mask_fill_fwd.  Returns ``None`` when unsupported (Q not a multiple of 8)."""
    x = _device_tensor(x, "input")
    if x.dim() != 4 or not x.is_contiguous():
        raise ValueError(f"expected a contiguous (N,C,P,Q) tensor, got {tuple(x.shape)}")
    n, c, p, q = x.shape
    visible = _device_tensor(visible, "visible")
    if visible.dtype == torch.bool:
        visible = visible.view(torch.uint8)
    if (visible.dtype != torch.uint8 or visible.dim() != 4 or not visible.is_contiguous() or visible.shape[2:] != (p, q)
            or visible.size(0) not in (1, n) or visible.size(1) not in (1, c)):
        raise ValueError(f"visible must be a contiguous uint8 / bool tensor of shape (1|{n}, 1|{c}, {p}, {q}), got "
                         f"{visible.dtype} {tuple(visible.shape)}")
    if visible.data_ptr() % 8 != 0:
        return None
    y = x if out is x else _out_like(x, out)
    with torch.cuda.device(x.device):
        rc = _lib.load().mta_mask_fill_fwd(x.data_ptr(), visible.data_ptr(), y.data_ptr(), n, c, p, q, visible.size(0),
                                           visible.size(1), int(bool(neg_inf)), int(bool(causal)), _code(x, "input"),
                                           _stream(x))
    if rc == _lib.MTA_ERR_UNSUPPORTED:
        return None
    _lib.check(rc, "mta_mask_fill_fwd")
    return y


def mask_add(x: torch.Tensor, mask: torch.Tensor, causal: bool, out: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """``x + mask`` in x's dtype for an additive mask of x's dtype and shape (1|N, 1|C, P, Q); with ``causal`` only keys
    q <= p are read and written.  ``out`` may be ``x``.  See mta_mask_add_fwd.  Returns ``None`` when unsupported."""
    x = _device_tensor(x, "input")
    if x.dim() != 4 or not x.is_contiguous():
        raise ValueError(f"expected a contiguous (N,C,P,Q) tensor, got {tuple(x.shape)}")
    n, c, p, q = x.shape
    mask = _device_tensor(mask, "mask")
    if (mask.dtype != x.dtype or mask.dim() != 4 or not mask.is_contiguous() or mask.shape[2:] != (p, q)
            or mask.size(0) not in (1, n) or mask.size(1) not in (1, c)):
        raise ValueError(f"mask must be a contiguous {x.dtype} tensor of shape (1|{n}, 1|{c}, {p}, {q}), got "
                         f"{mask.dtype} {tuple(mask.shape)}")
    if mask.data_ptr() % 16 != 0:
        return None
    y = x if out is x else _out_like(x, out)
    with torch.cuda.device(x.device):
        rc = _lib.load().mta_mask_add_fwd(x.data_ptr(), mask.data_ptr(), y.data_ptr(), n, c, p, q, mask.size(0),
                                          mask.size(1), int(bool(causal)), _code(x, "input"), _stream(x))
    if rc == _lib.MTA_ERR_UNSUPPORTED:
        return None
    _lib.check(rc, "mta_mask_add_fwd")
    return y


def causal_ptx(p: torch.Tensor, x: torch.Tensor, causal: bool) -> Optional[torch.Tensor]:
    """P^T X for P (B,H,S,S), X (B,H,S,D): out[k] = sum_p P[p,k] X[p], over p >= k only when causal (nothing of P above
    the diagonal is read); see mta_causal_ptx_fwd.  Returns ``None`` when unsupported (the caller then uses
    torch.matmul on a fully defined P)."""
    p = _device_tensor(p, "P")
    x = _device_tensor(x, "X")
    if p.dim() != 4 or x.dim() != 4 or p.shape[:3] != x.shape[:3] or p.shape[2] != p.shape[3] or p.dtype != x.dtype:
        return None
    b, h, s, d = x.shape
    out = torch.empty_like(x)
    with torch.cuda.device(p.device):
        rc = _lib.load().mta_causal_ptx_fwd(p.data_ptr(), x.data_ptr(), out.data_ptr(), b, h, s, d, int(bool(causal)),
                                            _code(p, "P"), _stream(p))
    if rc in (_lib.MTA_ERR_UNSUPPORTED, -7):
        return None
    _lib.check(rc, "mta_causal_ptx_fwd")
    return out


def causal_pv_supported(p_dtype: torch.dtype, s: int, d: int) -> bool:
    return p_dtype in (torch.bfloat16, torch.float16) and d in (64, 128) and s % 8 == 0


# ---------------------------------------------------------------------------------------
# weight structure probes (evaluated on the device; the result comes back in one small copy)
# ---------------------------------------------------------------------------------------
def _probe_head_into(weight: torch.Tensor, out: torch.Tensor) -> None:
    w = _device_tensor(weight.detach(), "weight")
    assert w.dim() == 2 and w.shape[0] == w.shape[1], f"Weight must be square matrix, got {w.shape}"
    with torch.cuda.device(w.device):
        rc = _lib.load().mta_probe_head_weight(w.data_ptr(), w.shape[0], _code(w, "weight"), out.data_ptr(), _stream(w))
    _lib.check(rc, "mta_probe_head_weight")


def _probe_conv_into(weight: torch.Tensor, out: torch.Tensor) -> None:
    w = _device_tensor(weight.detach(), "weight")
    assert w.dim() == 3, f"conv kernel must be (C,R,S), got {tuple(w.shape)}"
    with torch.cuda.device(w.device):
        rc = _lib.load().mta_probe_conv_kernel(w.data_ptr(), w.shape[0], w.shape[1], w.shape[2], _code(w, "weight"),
                                               out.data_ptr(), _stream(w))
    _lib.check(rc, "mta_probe_conv_kernel")


def probe_head_weight(weight: torch.Tensor):
    """(is exactly the identity, smallest G such that the (H,H) weight is zero outside its GxG diagonal blocks)."""
    out = torch.empty(2, dtype=torch.int32, device=weight.device)
    _probe_head_into(weight, out)
    eye, group = out.tolist()
    return bool(eye), int(group)


def probe_conv_kernel(weight: torch.Tensor) -> bool:
    """True when the (C,R,S) kernel is exactly 1.0 at [R-1, S//2] and 0 elsewhere, S odd (a pass-through)."""
    out = torch.empty(1, dtype=torch.int32, device=weight.device)
    _probe_conv_into(weight, out)
    return bool(out.item())


def probe_mta_weights(w_pre: torch.Tensor, w_post: torch.Tensor, conv_post: torch.Tensor):
    """The three probes the MTA glue needs, with a single read back:
    (pre identity, pre group, post identity, post group, post conv identity)."""
    out = torch.empty(5, dtype=torch.int32, device=w_pre.device)
    _probe_head_into(w_pre, out[0:2])
    _probe_head_into(w_post, out[2:4])
    _probe_conv_into(conv_post, out[4:5])
    a, b, c, d, e = out.tolist()
    return bool(a), int(b), bool(c), int(d), bool(e)
