"""GPU parity of the backward entry points (through the C ABI) against torch.autograd through the CPU oracle.

  mta_conv2d_bwd_input / _weight     vs oracle.depthwise_conv_grads   (convolution_2d_trit.py:143-295, 336-378)
  mta_headmix_bwd_input / _weight    vs oracle.head_linear_grads      (triton_linear_head.py:144-278, 322-370)
  MTAAttentionTriton(...).backward() vs autograd through oracle.mta_forward: the gradient checks of the
                                     reference's compare script (compare_mta_attention.py:123-162)

Tolerances.  fp32: rtol 1e-4, atol 1e-5 times the largest expected magnitude (weight gradients are sums over
up to 10^6 products, so the absolute floor scales with them).  bf16/fp16: inputs and the input gradient are
stored in 16 bits: 2e-2 times the largest expected magnitude; weight gradients are accumulated and returned
in fp32 from 16-bit inputs that the oracle sees as the same 16-bit values, so they keep rtol 1e-3.
Softmax gradients of 16-bit data are small numbers (|dx| <= p |dp - sum|, p of the order 1 / row length), which an
absolute bar never reaches: they are compared element by element with the value the same rounded probabilities give
(`_softmax_grad_close`).  Module gradients in 16 bits also meet a bar on the relative error norm per tensor
(`_rel_norm`): what the oracle's own pipeline run in that dtype on the CPU deviates from its fp32 run is 0.5-0.8 %
(bf16) and 0.06-0.09 % (fp16); the bars are 2 % and 0.4 %.
"""
import pytest
import torch

from oracle import mta_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pkg():
    import multitokenatention_triton_amd as m
    return m


def _close(got, want, dtype, what, weight_grad=False):
    got, want = got.detach().cpu().float(), want.detach().cpu().float()
    scale = max(1.0, float(want.abs().max()))
    if dtype == torch.float32:
        torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-5 * scale, msg=lambda m: f"{what}: {m}")
    elif weight_grad:
        torch.testing.assert_close(got, want, rtol=1e-3, atol=1e-3 * scale, msg=lambda m: f"{what}: {m}")
    else:
        torch.testing.assert_close(got, want, rtol=0.0, atol=2e-2 * scale, msg=lambda m: f"{what}: {m}")


def _rel_norm(got, want, dtype, what):
    """||got - want|| / ||want|| per tensor: a bar that an all-zero or a half-wrong result cannot pass."""
    got, want = got.detach().cpu().float(), want.detach().cpu().float()
    bar = {torch.float32: 1e-4, torch.bfloat16: 2e-2, torch.float16: 4e-3}[dtype]
    rel = float((got - want).norm() / want.norm().clamp_min(1e-30))
    assert rel < bar, f"{what}: relative error norm {rel:.3e} >= {bar:.0e}"


def _softmax_grad_close(got, p16, dp, up, dtype, what):
    """dx = p (dp - sum_k p dp) from the probabilities as the kernel sees them (rounded to the score dtype).  The kernel
    works in fp32 and rounds once: |got - want| <= one unit in the last place of want (2^-8 / 2^-11 relative) + p times
    the fp32 summation error of the bracket + half a subnormal step of the format."""
    p = p16.detach().cpu().float()
    g = dp.detach().cpu().float()
    if up is not None:
        p, g = p.masked_fill(up, 0.0), g.masked_fill(up, 0.0)
    dot = (p * g).sum(-1, keepdim=True)
    absdot = (p * g.abs()).sum(-1, keepdim=True)
    want = p * (g - dot)
    got = got.detach().cpu().float()
    if dtype == torch.float32:
        bound = 1e-4 * want.abs() + p * 1e-5 * (g.abs() + absdot) + 1e-30
    else:
        ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
        tiny = 0.0 if dtype == torch.bfloat16 else 2.0 ** -24
        bound = ulp * want.abs() + p * 1e-5 * (g.abs() + absdot) + tiny + 1e-30
    bad = (got - want).abs() > bound
    assert not bad.any(), (f"{what}: {int(bad.sum())} of {bad.numel()} entries off; worst "
                           f"{float(((got - want).abs() - bound).max()):.3e} beyond its bound")
    assert float(got.abs().sum()) >= 0.5 * float(want.abs().sum())   # (not an all-zero result)


def _rand(shape, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g).to(dtype)


CONV_CASES = [
    # N, C, H, W, R, S, causal
    (2, 3, 40, 40, 3, 3, True),
    (1, 2, 100, 100, 6, 11, True),
    (1, 2, 70, 70, 6, 11, False),
    (2, 2, 33, 65, 5, 7, False),       # ragged, not square
    (1, 2, 257, 257, 3, 5, True),      # width not a multiple of 8
    (1, 1, 1, 1, 3, 3, True),
    (1, 2, 64, 64, 2, 4, True),        # even key size, no fixed-size instance
    (1, 1, 48, 48, 11, 15, True),      # general kernels
    (1, 2, 264, 264, 7, 7, True),
    (1, 2, 512, 512, 6, 11, True),     # several strips / tiles per plane, interior ones included
    (1, 1, 200, 200, 7, 9, True),
    # 16-bit: matrix-core weight-gradient kernel (rows of whole 16-byte vectors)
    (1, 2, 72, 72, 6, 11, False),
    (2, 2, 40, 96, 5, 5, False),       # not square
    (1, 2, 96, 40, 3, 5, True),        # causal rule on a tall plane: keys beyond the row index never take part
    (1, 1, 1040, 1040, 7, 7, True),    # key range cut into segments, many steps per item
    (3, 5, 136, 136, 5, 7, True),
    (1, 1, 80, 80, 77, 77, True),      # the largest kernel of the reference's published rows
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", CONV_CASES)
def test_conv_backward_parity(pkg, case, dtype):
    n, c, h, w, r, s, causal = case
    print(f"conv bwd case={case} {dtype}", flush=True)
    x, dy = _rand((n, c, h, w), 1, dtype), _rand((n, c, h, w), 2, dtype)
    wt = (0.2 * _rand((c, r, s), 3, torch.float32)).to(dtype)
    if causal and h == w:   # what lies above the diagonal must never be read
        up = torch.triu(torch.ones(h, w, dtype=torch.bool), 1)
        x_dev, dy_dev = x.masked_fill(up, float("nan")).cuda(), dy.masked_fill(up, float("nan")).cuda()
    else:
        x_dev, dy_dev = x.cuda(), dy.cuda()
    want_dx, want_dw = O.depthwise_conv_grads(x.float(), wt.float(), causal, dy.float())
    dx = pkg.ops.conv2d_bwd_input(dy_dev, wt.cuda(), causal)
    dw = pkg.ops.conv2d_bwd_weight(x_dev, dy_dev, (r, s), causal)
    assert dx.dtype == dtype and dx.shape == x.shape and dw.dtype == torch.float32 and dw.shape == (c, r, s)
    _close(dx, want_dx, dtype, "dx")
    _close(dw, want_dw, dtype, "dw", weight_grad=True)
    if causal and h == w:
        up = torch.triu(torch.ones(h, w, dtype=torch.bool), 1)
        assert (dx.cpu()[..., up] == 0).all() and not torch.signbit(dx.cpu()[..., up]).any()
    # run to run bit-reproducible
    assert torch.equal(dw, pkg.ops.conv2d_bwd_weight(x_dev, dy_dev, (r, s), causal))


def test_conv_backward_full_size(pkg):
    """BASELINE config 2 at full size, (2,16,2048,2048) bf16 6x11 causal: the kernel gradient of every channel is the sum
    of the two batch elements' (linearity, all channels), and two channels are compared with the oracle on their own
    slices; the input gradient of those channels likewise."""
    print("conv bwd full size", flush=True)
    n, c, s, r, sk = 2, 16, 2048, 6, 11
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(71)
    x = torch.tril(torch.randn(n, c, s, s, generator=g).to(dtype))
    dy = torch.tril(torch.randn(n, c, s, s, generator=g).to(dtype))
    wt = (0.2 * torch.randn(c, r, sk, generator=g)).to(dtype)
    xd, dyd = x.cuda(), dy.cuda()
    dw = pkg.ops.conv2d_bwd_weight(xd, dyd, (r, sk), True)
    parts = sum(pkg.ops.conv2d_bwd_weight(xd[b:b + 1].contiguous(), dyd[b:b + 1].contiguous(), (r, sk), True) for b in range(n))
    _close(dw, parts, dtype, "dw = sum over the batch", weight_grad=True)
    dx = pkg.ops.conv2d_bwd_input(dyd, wt.cuda(), True)
    for ch in (3, 12):
        want_dx, want_dw = O.depthwise_conv_grads(x[:, ch:ch + 1].float(), wt[ch:ch + 1].float(), True, dy[:, ch:ch + 1].float())
        _close(dw[ch:ch + 1], want_dw, dtype, f"dw channel {ch}", weight_grad=True)
        _close(dx[:, ch:ch + 1], want_dx, dtype, f"dx channel {ch}")


HM_CASES = [
    # N, C, P, Q, group, causal
    (2, 4, 40, 40, None, True),
    (1, 16, 136, 136, None, True),     # matrix-core weight-gradient kernel (16-bit)
    (1, 32, 264, 264, None, True),
    (2, 32, 128, 128, None, False),
    (1, 16, 100, 100, 4, True),        # width not a multiple of 8
    (1, 8, 72, 72, 2, True),
    (1, 6, 33, 65, None, False),
    (1, 16, 300, 304, None, False),
    (1, 1, 1, 1, None, True),
    (1, 48, 64, 64, None, True),
    (1, 64, 136, 136, None, True),     # wide matrix-core mixing kernel with the transposed matrix (input gradient)
    (1, 128, 72, 264, None, False),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", HM_CASES)
def test_headmix_backward_parity(pkg, case, dtype):
    n, c, p, q, group, causal = case
    print(f"headmix bwd case={case} {dtype}", flush=True)
    x, dy = _rand((n, c, p, q), 4, dtype), _rand((n, c, p, q), 5, dtype)
    g = torch.Generator().manual_seed(6)
    if group:
        wt = O.block_diag_head_weight(c, group, 0.3, g, dtype)
    else:
        wt = (torch.eye(c) + 0.3 * torch.randn(c, c, generator=g)).to(dtype)
    if causal and p == q:
        up = torch.triu(torch.ones(p, q, dtype=torch.bool), 1)
        x_dev, dy_dev = x.masked_fill(up, float("nan")).cuda(), dy.masked_fill(up, float("nan")).cuda()
    else:
        x_dev, dy_dev = x.cuda(), dy.cuda()
    want_dx, want_dw = O.head_linear_grads(x.float(), wt.float(), causal, 0.0, dy.float())
    dx = pkg.ops.headmix_bwd_input(dy_dev, wt.cuda(), causal, group_size=group)
    dw = pkg.ops.headmix_bwd_weight(x_dev, dy_dev, causal)
    assert dx.dtype == dtype and dw.dtype == torch.float32 and dw.shape == (c, c)
    _close(dx, want_dx, dtype, "dx")
    _close(dw, want_dw, dtype, "dw", weight_grad=True)
    if causal and p == q:
        assert (dx.cpu()[..., up] == 0).all()
    assert torch.equal(dw, pkg.ops.headmix_bwd_weight(x_dev, dy_dev, causal))


SM_CASES = [
    # N, C, P, Q, causal
    (1, 2, 40, 40, True),
    (2, 3, 264, 264, True),        # rows of whole 16-byte vectors: one read of p and dp
    (1, 2, 100, 104, False),
    (1, 1, 33, 65, False),         # ragged
    (1, 2, 2304, 2304, True),      # two vectors per thread
    (1, 1, 300, 4360, False),      # four vectors per thread
    (1, 1, 3, 8200, False),        # longer than the register path holds
    (1, 1, 1, 1, True),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", SM_CASES)
def test_softmax_backward_parity(pkg, case, dtype):
    """mta_softmax_bwd against torch.autograd through F.softmax(x.float()).type_as(x), the expression the reference
    differentiates (mta_attention_triton.py:79).  The kernel sees the probabilities rounded to the score dtype, autograd
    their fp32 originals: for 16-bit data the bar is atol 2e-2 * max|dx| (each rounded p is within 2^-9 of its
    original); fp32: rtol 1e-4.  Above the diagonal: +0 with fill_upper, untouched without."""
    n, c, rows, q, causal = case
    print(f"softmax bwd case={case} {dtype}", flush=True)
    x, dp = _rand((n, c, rows, q), 5, dtype), _rand((n, c, rows, q), 6, dtype)
    up = torch.triu(torch.ones(rows, q, dtype=torch.bool), 1)
    leaf = x.float().masked_fill(up, float("-inf")) if causal else x.float()
    leaf.requires_grad_(True)
    probs = torch.softmax(leaf, -1)
    probs.backward(dp.float().masked_fill(up, 0.0) if causal else dp.float())
    want = leaf.grad
    p_dev, dp_dev = probs.detach().to(dtype).cuda(), dp.cuda()
    if causal:   # what lies above the diagonal must never be read
        p_dev, dp_dev = p_dev.masked_fill(up.cuda(), float("nan")), dp_dev.masked_fill(up.cuda(), float("nan"))
    got = pkg.ops.softmax_bwd(p_dev, dp_dev, causal)
    assert got.dtype == dtype and got.shape == x.shape
    _close(got, want, dtype, "dx")
    _softmax_grad_close(got, probs.detach().to(dtype), dp, up if causal else None, dtype, "dx from the rounded p")
    if causal:
        g = got.cpu()
        assert (g[..., up] == 0).all() and not torch.signbit(g[..., up]).any()
        # fill_upper=False: the same below the diagonal, nothing written in vectors wholly above it
        sentinel = torch.full_like(p_dev, 7.0)
        lib = pkg._lib.load()
        rc = lib.mta_softmax_bwd(p_dev.data_ptr(), dp_dev.data_ptr(), sentinel.data_ptr(), n, c, rows, q, 1, 0,
                                 {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}[dtype],
                                 torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        low = ~up
        assert torch.equal(sentinel.cpu()[..., low], g[..., low])
        far = torch.triu(torch.ones(rows, q, dtype=torch.bool), 8)   # beyond any vector that touches the diagonal
        assert (sentinel.cpu()[..., far] == 7.0).all()


def test_headmix_and_softmax_backward_full_size(pkg):
    """(2,32,2048,2048) bf16, BASELINE config 3's shape: the head-mixing weight gradient is the sum of the two batch
    elements' (linearity) and symmetric in its arguments (dW(x, dy) = dW(dy, x)^T); the softmax gradient, whose rows are
    independent, is compared with autograd on slabs of rows of two planes."""
    print("headmix / softmax bwd full size", flush=True)
    n, c, s = 2, 32, 2048
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(72)
    xd = torch.randn(n, c, s, s, generator=g).to(dtype).cuda()
    dyd = torch.randn(n, c, s, s, generator=g).to(dtype).cuda()
    dw = pkg.ops.headmix_bwd_weight(xd, dyd, True)
    parts = sum(pkg.ops.headmix_bwd_weight(xd[b:b + 1].contiguous(), dyd[b:b + 1].contiguous(), True) for b in range(n))
    _close(dw, parts, dtype, "dw = sum over the batch", weight_grad=True)
    _close(pkg.ops.headmix_bwd_weight(dyd, xd, True).t(), dw, dtype, "dw(dy, x)^T", weight_grad=True)
    # softmax gradient: p from the CPU softmax of the same logits, rows 0-63 and the last 96 of planes (0,5) and (1,30)
    up = torch.triu(torch.ones(s, s, dtype=torch.bool), 1)
    for b, ch in ((0, 5), (1, 30)):
        logits = xd[b, ch].cpu().float().masked_fill(up, float("-inf")).requires_grad_(True)
        probs = torch.softmax(logits, -1)
        probs.backward(dyd[b, ch].cpu().float().masked_fill(up, 0.0))
        p_dev = torch.zeros(1, 1, s, s, dtype=dtype, device="cuda")
        p_dev[0, 0] = probs.detach().to(dtype).cuda()
        got = pkg.ops.softmax_bwd(p_dev, dyd[b:b + 1, ch:ch + 1].contiguous(), True)[0, 0].cpu()
        for rows in (slice(0, 64), slice(s - 96, s)):
            _close(got[rows], logits.grad[rows], dtype, f"softmax dx plane {(b, ch)} rows {rows}")
            _softmax_grad_close(got[rows], probs.detach().to(dtype)[rows], dyd[b, ch].cpu()[rows], up[rows], dtype,
                                f"softmax dx from the rounded p, plane {(b, ch)} rows {rows}")


def test_operator_functions_backward(pkg):
    """Conv2dTritonFunction / TritonLinearHeadFunction under torch.autograd, fp32, against the oracle's grads."""
    print("operator Functions backward", flush=True)
    x = _rand((1, 4, 50, 50), 7, torch.float32)
    dy = _rand((1, 4, 50, 50), 8, torch.float32)
    w = 0.2 * _rand((4, 3, 5), 9, torch.float32)
    conv = pkg.Conv2dTriton(4, (3, 5), causal=True).cuda()
    with torch.no_grad():
        conv.weight.copy_(w)
    xd = x.cuda().requires_grad_(True)
    conv(xd).backward(dy.cuda())
    want_dx, want_dw = O.depthwise_conv_grads(x, w, True, dy)
    _close(xd.grad, want_dx, torch.float32, "conv dx")
    _close(conv.weight.grad, want_dw, torch.float32, "conv dw")

    g = torch.Generator().manual_seed(10)
    wm = O.block_diag_head_weight(4, 2, 0.3, g)
    for group in (None, 2):
        lin = pkg.TritonLinearHead(4, causal=True, output_value=float("-inf"), group_size=group).cuda()
        with torch.no_grad():
            lin.weight.copy_(wm)
        xd = x.cuda().requires_grad_(True)
        y = lin(xd)
        assert torch.isneginf(y[0, 0, 0, 1])
        y.backward(dy.cuda())
        want_dx, want_dw = O.head_linear_grads(x, wm, True, float("-inf"), dy)
        _close(xd.grad, want_dx, torch.float32, "headmix dx")
        if group:   # the gradient is confined to the declared blocks
            blk = torch.arange(4) // group
            want_dw = want_dw * (blk[:, None] == blk[None, :])
        _close(lin.weight.grad, want_dw, torch.float32, "headmix dw")


def _mta_pair(pkg, h, r1, s1, dtype, seed, causal=True):
    g = torch.Generator().manual_seed(seed)
    params = [O.seeded_conv_weight(h, r1, s1, 0.1, torch.float32, seed=seed + 1),
              torch.eye(h) + 0.1 * torch.randn(h, h, generator=g),
              O.seeded_conv_weight(h, 3, 3, 0.1, torch.float32, seed=seed + 2),
              torch.eye(h) + 0.1 * torch.randn(h, h, generator=g)]
    params = [p.to(dtype) for p in params]
    cfg = pkg.MTAConfig(query_kernel_size=r1, key_kernel_size=s1)
    mod = pkg.MTAAttentionTriton(h, cfg, dropout=0.0, causal=causal)
    with torch.no_grad():
        for dst, src in zip((mod.mta_conv_triton, mod.wpsm_triton, mod.mta_conv_after_sm_triton, mod.wposm_triton), params):
            dst.weight.copy_(src)
    return mod.to(dtype).cuda().eval(), params


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_mta_module_backward(pkg, dtype):
    """compare_mta_attention.py:123-162 restated: gradients with respect to xq, xk, xv and the four MTA weights of
    MTAAttentionTriton against autograd through the PyTorch restatement (seed 123, B2 H16 S128 D64 as in :21-27,
    with non-trivial weights so that every gradient is exercised)."""
    print(f"mta module backward {dtype}", flush=True)
    b, h, s, d = 2, 16, 128, 64
    mod, params = _mta_pair(pkg, h, 3, 3, dtype, seed=123)
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=123)
    go = _rand((b, s, h, d), 124, dtype)

    # oracle, fp32 arithmetic on the same 16-bit values
    leaves = [t.detach().clone().float().requires_grad_(True) for t in (q, k, v)]
    wl = [p.detach().clone().float().requires_grad_(True) for p in params]
    out = O.mta_forward(*leaves, wl[0].unsqueeze(1), wl[1], wl[2].unsqueeze(1), wl[3])
    out.backward(go.float())

    qd, kd, vd = [t.detach().clone().cuda().requires_grad_(True) for t in (q, k, v)]
    got = mod(qd, kd, vd, None, None)
    assert got.requires_grad
    _close(got, out, dtype, "forward")
    got.backward(go.cuda())
    for name, gt, wt in (("xq", qd.grad, leaves[0].grad), ("xk", kd.grad, leaves[1].grad), ("xv", vd.grad, leaves[2].grad)):
        assert gt is not None and gt.dtype == dtype
        _close(gt, wt, dtype, f"grad {name}")
        _rel_norm(gt, wt, dtype, f"grad {name}")
    for name, p_, wt in (("pre conv", mod.mta_conv_triton.weight, wl[0].grad), ("wpsm", mod.wpsm_triton.weight, wl[1].grad),
                         ("post conv", mod.mta_conv_after_sm_triton.weight, wl[2].grad),
                         ("wposm", mod.wposm_triton.weight, wl[3].grad)):
        assert p_.grad is not None and p_.grad.dtype == dtype
        # (intermediate score tensors are stored in 16 bits along the way: the element bar is the 16-bit one, on sums
        # of magnitude ~100; the norm bar is what pins them)
        _close(p_.grad, wt, dtype, f"grad {name}")
        _rel_norm(p_.grad, wt, dtype, f"grad {name}")


@pytest.mark.parametrize("shape", [(1, 8, 100, 32, 6, 11), (2, 4, 264, 128, 7, 7), (1, 32, 136, 64, 3, 5)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_mta_module_backward_other_shapes(pkg, shape, dtype):
    """The training route where its single-kernel stages do not apply and where they do: a head size and a sequence
    length without a scores kernel (library GEMM + scaled conv, GEMM for dP), 8 heads (packed mix + softmax), 32 dense
    heads (mixing and softmax as two kernels), head size 128 with a 7x7 kernel."""
    b, h, s, d, r1, s1 = shape
    print(f"mta module backward shape={shape} {dtype}", flush=True)
    mod, params = _mta_pair(pkg, h, r1, s1, dtype, seed=321)
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=322)
    go = _rand((b, s, h, d), 323, dtype)
    leaves = [t.detach().clone().float().requires_grad_(True) for t in (q, k, v)]
    wl = [p.detach().clone().float().requires_grad_(True) for p in params]
    out = O.mta_forward(*leaves, wl[0].unsqueeze(1), wl[1], wl[2].unsqueeze(1), wl[3])
    out.backward(go.float())
    qd, kd, vd = [t.detach().clone().cuda().requires_grad_(True) for t in (q, k, v)]
    got = mod(qd, kd, vd, None, None)
    _close(got, out, dtype, "forward")
    got.backward(go.cuda())
    for name, gt, wt in (("xq", qd.grad, leaves[0].grad), ("xk", kd.grad, leaves[1].grad), ("xv", vd.grad, leaves[2].grad)):
        _close(gt, wt, dtype, f"grad {name}")
        _rel_norm(gt, wt, dtype, f"grad {name}")
    for name, p_, wt in (("pre conv", mod.mta_conv_triton.weight, wl[0].grad), ("wpsm", mod.wpsm_triton.weight, wl[1].grad),
                         ("post conv", mod.mta_conv_after_sm_triton.weight, wl[2].grad),
                         ("wposm", mod.wposm_triton.weight, wl[3].grad)):
        _close(p_.grad, wt, dtype, f"grad {name}")
        _rel_norm(p_.grad, wt, dtype, f"grad {name}")


def test_mta_module_backward_reference_bar(pkg):
    """The reference script's own configuration and bar: identity parameters after reset_mta_parameters(), fp32,
    allclose(rtol=1e-3, atol=1e-5) on the three input gradients (compare_mta_attention.py:21-27, 60-74, 113, 136-138)."""
    print("mta module backward, reference bar", flush=True)
    b, h, s, d = 2, 16, 128, 64
    mod = pkg.MTAAttentionTriton(h, pkg.MTAConfig(), 0.0, True).cuda().eval()
    mod.reset_mta_parameters()
    q, k, v = O.seeded_qkv(b, h, s, d, torch.float32, seed=123)
    go = _rand((b, s, h, d), 125, torch.float32)
    leaves = [t.clone().requires_grad_(True) for t in (q, k, v)]
    want = torch.nn.functional.scaled_dot_product_attention(*leaves, is_causal=True).transpose(1, 2)
    want.backward(go)
    qd, kd, vd = [t.detach().clone().cuda().requires_grad_(True) for t in (q, k, v)]
    got = mod(qd, kd, vd, None, None)
    got.backward(go.cuda())
    for gt, wt in ((qd.grad, leaves[0].grad), (kd.grad, leaves[1].grad), (vd.grad, leaves[2].grad)):
        torch.testing.assert_close(gt.cpu(), wt, rtol=1e-3, atol=1e-5)
    for p_ in mod.parameters():
        assert p_.grad is not None and torch.isfinite(p_.grad).all()


def test_mta_module_backward_with_mask(pkg):
    """use_mask=True trains through the same operator Functions."""
    print("mta module backward use_mask", flush=True)
    b, h, s, d = 1, 4, 72, 64
    dtype = torch.float32
    mod, params = _mta_pair(pkg, h, 3, 5, dtype, seed=321)
    mod.use_mask = True
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=322)
    keep = torch.ones(1, s, dtype=torch.bool)
    keep[0, 5:9] = False
    go = _rand((b, s, h, d), 323, dtype)
    leaves = [t.clone().requires_grad_(True) for t in (q, k, v)]
    wl = [p.clone().requires_grad_(True) for p in params]
    out = O.mta_forward(*leaves, wl[0].unsqueeze(1), wl[1], wl[2].unsqueeze(1), wl[3], mask=keep)
    out.backward(go)
    qd, kd, vd = [t.detach().clone().cuda().requires_grad_(True) for t in (q, k, v)]
    got = mod(qd, kd, vd, keep.cuda(), None)
    _close(got, out, dtype, "forward")
    got.backward(go.cuda())
    _close(qd.grad, leaves[0].grad, dtype, "grad xq")
    _close(kd.grad, leaves[1].grad, dtype, "grad xk")
    _close(vd.grad, leaves[2].grad, dtype, "grad xv")
    _close(mod.mta_conv_triton.weight.grad, wl[0].grad, dtype, "grad pre conv")
    _close(mod.wposm_triton.weight.grad, wl[3].grad, dtype, "grad wposm")


# ------------------------------------------------------------------------------------------------------
# the pieces that exist only on the 16-bit training route, and that route at the sizes the benchmark times
# ------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_lower_scores_is_the_rounded_product(pkg, d, dtype):
    """_lower_scores(a, b) = round(a b^T) on and below the diagonal (the scores kernel with factor 1 and the pass-through
    tap as 3x3 kernel; the training route's dP = dO V^T and its recomputed raw scores).  (1) Operands of small integers:
    every partial sum and the result are exact in fp32 and in the 16-bit type, so the result is the product bit for bit
    whatever the order of summation - a conv stage that did anything but copy would show.  (2) N(0,1) operands: within
    one unit in the last place of the fp64 product (fp32 accumulation in another order, then one rounding; 1e-4 absolute
    for entries that cancel to almost nothing), and equal to it on all but a few entries.  (3) The same call into a buffer that holds NaN: the lower triangle is unchanged."""
    from multitokenatention_triton_amd.mta_attention_triton import _lower_scores
    print(f"_lower_scores d={d} {dtype}", flush=True)
    b, h, s = 1, 3, 520
    g = torch.Generator().manual_seed(11)
    low = torch.tril(torch.ones(s, s, dtype=torch.bool))
    a = torch.randint(-1, 2, (b, h, s, d), generator=g).to(dtype)
    c = torch.randint(-1, 2, (b, h, s, d), generator=g).to(dtype)
    got = _lower_scores(a.cuda(), c.cuda())
    assert got is not None and got.dtype == dtype and got.shape == (b, h, s, s)
    want = torch.matmul(a.float(), c.float().transpose(2, 3)).to(dtype)
    assert torch.equal(got.cpu()[..., low], want[..., low])

    a, c = _rand((b, h, s, d), 12, dtype), _rand((b, h, s, d), 13, dtype)
    got = _lower_scores(a.cuda(), c.cuda()).cpu()
    exact = torch.matmul(a.double(), c.double().transpose(2, 3))
    want = exact.to(dtype)
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
    diff = (got.double() - want.double()).abs()[..., low]
    assert (diff <= ulp * exact.abs()[..., low] + 1e-4).all()   # (+ the fp32 accumulation error of up to 128 terms)
    assert float((diff == 0).double().mean()) > 0.99

    w = torch.zeros(h, 3, 3, dtype=dtype)
    w[:, 2, 1] = 1.0
    buf = torch.full((b, h, s, s), float("nan"), dtype=dtype, device="cuda")
    out = pkg.ops.qk_conv(a.cuda(), c.cuda(), w.cuda(), True, 1.0, fill_upper=False, out=buf)
    assert out is buf and torch.equal(buf.cpu()[..., low], got[..., low])

    # under a band mask: the same products inside the band, exact zeros ahead of it - also where the kernel skips whole
    # key blocks (a window much shorter than the rows)
    rows = torch.arange(s)
    first = (rows - 70).clamp(min=0).to(torch.int32)
    first[300:] = 290
    got_band = _lower_scores(a.cuda(), c.cuda(), first[None].expand(b, s).contiguous().cuda()).cpu()
    inside = low & (torch.arange(s)[None, :] >= first[:, None])
    assert torch.equal(got_band[..., inside], got[..., inside])
    assert not got_band[..., low & ~inside].any()


def _oracle_grads(q, k, v, params, go, mask=None):
    leaves = [t.detach().clone().float().requires_grad_(True) for t in (q, k, v)]
    wl = [p.detach().clone().float().requires_grad_(True) for p in params]
    out = O.mta_forward(*leaves, wl[0].unsqueeze(1), wl[1], wl[2].unsqueeze(1), wl[3], mask=mask)
    out.backward(go.float())
    return out.detach(), [t.grad for t in leaves], [t.grad for t in wl]


def _module_grads(mod, q, k, v, go, mask=None):
    qd, kd, vd = [t.detach().clone().cuda().requires_grad_(True) for t in (q, k, v)]
    for p_ in mod.parameters():
        p_.grad = None
    got = mod(qd, kd, vd, None if mask is None else mask.cuda(), None)
    got.backward(go.cuda())
    ws = (mod.mta_conv_triton.weight, mod.wpsm_triton.weight, mod.mta_conv_after_sm_triton.weight, mod.wposm_triton.weight)
    return got.detach(), [qd.grad, kd.grad, vd.grad], [w.grad for w in ws]


_GRAD_NAMES = ("xq", "xk", "xv", "pre conv", "wpsm", "post conv", "wposm")


def _check_all(dtype, out, want_out, grads, want_grads):
    _close(out, want_out, dtype, "forward")
    _rel_norm(out, want_out, dtype, "forward")
    for name, gt, wt in zip(_GRAD_NAMES, grads, want_grads):
        assert gt is not None and gt.dtype == dtype, name
        _close(gt, wt, dtype, f"grad {name}")
        _rel_norm(gt, wt, dtype, f"grad {name}")


@pytest.mark.parametrize("shape", [(1, 4, 2048, 128, 6, 11, torch.bfloat16), (1, 16, 1024, 128, 7, 7, torch.float16)])
def test_mta_module_backward_long_sequence(pkg, shape):
    """The training route at sequence lengths where its kernels run as they do at the benchmark shape: several work
    items per query block and a split key range in the scores kernel (forward, dP and the recomputed raw scores), rows of
    several passes in the softmax and its gradient, long key segments in the two weight-gradient kernels, dense 4 / 16
    head weights.  All seven gradients against autograd through the fp32 oracle on the same 16-bit values."""
    b, h, s, d, r1, s1, dtype = shape
    print(f"mta module backward long shape={shape}", flush=True)
    mod, params = _mta_pair(pkg, h, r1, s1, dtype, seed=331)
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=332)
    go = _rand((b, s, h, d), 333, dtype)
    want_out, want_in, want_w = _oracle_grads(q, k, v, params, go)
    stages = []
    mod._stage_hook = stages.append
    out, gin, gw = _module_grads(mod, q, k, v, go)
    assert stages[0] == "qk_conv" and "qk" not in stages
    _check_all(dtype, out, want_out, gin + gw, want_in + want_w)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mta_module_backward_non_causal(pkg, dtype):
    """MTAAttentionTriton(causal=False) in training: every stage and every gradient kernel in its unmasked form, chained;
    against autograd through the oracle with an all-visible mask."""
    print(f"mta module backward causal=False {dtype}", flush=True)
    b, h, s, d = 2, 4, 136, 64
    mod, params = _mta_pair(pkg, h, 3, 5, dtype, seed=341, causal=False)
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=342)
    go = _rand((b, s, h, d), 343, dtype)
    want_out, want_in, want_w = _oracle_grads(q, k, v, params, go, mask=torch.zeros(1, 1, s, s))
    out, gin, gw = _module_grads(mod, q, k, v, go)
    _check_all(dtype, out, want_out, gin + gw, want_in + want_w)


def test_mta_module_backward_key_mask_16bit(pkg):
    """use_mask=True with a key mask, bf16, in training (the mask tensor route through the operator Functions)."""
    print("mta module backward use_mask bf16", flush=True)
    dtype = torch.bfloat16
    b, h, s, d = 1, 4, 136, 64
    mod, params = _mta_pair(pkg, h, 3, 5, dtype, seed=351)
    mod.use_mask = True
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=352)
    keep = torch.ones(1, s, dtype=torch.bool)
    keep[0, 5:9] = False
    keep[0, 70] = False
    go = _rand((b, s, h, d), 353, dtype)
    want_out, want_in, want_w = _oracle_grads(q, k, v, params, go, mask=keep)
    out, gin, gw = _module_grads(mod, q, k, v, go, mask=keep)
    _check_all(dtype, out, want_out, gin + gw, want_in + want_w)


@pytest.mark.parametrize("case", [(3, 4, 264, 64, 3, 5, torch.bfloat16), (2, 16, 520, 128, 6, 11, torch.float16),
                                  (2, 8, 200, 64, 7, 7, torch.float32)])
def test_mta_module_backward_right_padded_batch(pkg, case):
    """Training under key padding for B > 1 (a (B,1,S,S) boolean mask: causal rule + hidden keys per batch entry): the mask
    is recognised and the differentiable operators run with a key bias and zeroed K and V rows - the first stage is the
    scores kernel, not a composite over (B,H,S,S) mask tensors.  All seven gradients against autograd through the oracle
    given the mask tensor; the K and V rows of the padding receive exactly zero."""
    b, h, s, d, r1, s1, dtype = case
    print(f"mta module backward right padding {case}", flush=True)
    mod, params = _mta_pair(pkg, h, r1, s1, dtype, seed=361)
    mod.use_mask = True
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=362)
    lengths = torch.tensor([s, s - s // 3, 41][:b])
    keep = torch.arange(s)[None, :] < lengths[:, None]
    visible = keep[:, None, None, :] & torch.tril(torch.ones(s, s, dtype=torch.bool))[None, None]
    go = _rand((b, s, h, d), 363, dtype)
    go = go * keep[:, :, None, None]   # (the padding rows' outputs are nobody's business)
    want_out, want_in, want_w = _oracle_grads(q, k, v, params, go, mask=visible.expand(b, h, s, s))
    stages = []
    mod._stage_hook = stages.append
    out, gin, gw = _module_grads(mod, q, k, v, go, mask=visible)
    if (r1, s1, d) == (6, 11, 128):   # (a size the scores kernel is built for)
        assert "qk_conv" in stages, stages
    assert "pv" in stages and ("mix_softmax" in stages or "softmax" in stages), stages
    real = keep[:, None, :, None]
    _check_all(dtype, out.cpu() * keep[:, :, None, None], want_out * keep[:, :, None, None], [g.cpu() for g in gin + gw], want_in + want_w)
    for name, g in (("xk", gin[1]), ("xv", gin[2])):
        assert not (g.cpu() * ~real).any(), f"grad {name} of a hidden key is not zero"


def _band_masks(s):
    rows = torch.arange(s)
    lower = rows[None, :] <= rows[:, None]
    window = lower & (rows[:, None] - rows[None, :] < 37)
    starts = torch.tensor([0, 50, 51, 130, s - 3])
    doc = (rows[:, None] >= starts[None, :]).sum(-1) - 1          # document of every position
    documents = lower & (doc[:, None] == doc[None, :])
    return {"window": window, "documents": documents}


@pytest.mark.parametrize("kind", ["window", "documents"])
@pytest.mark.parametrize("case", [(2, 4, 264, 64, 3, 3, torch.bfloat16), (1, 16, 520, 128, 6, 11, torch.float16),
                                  (2, 8, 200, 64, 7, 7, torch.bfloat16)])
def test_mta_module_backward_band_masks(pkg, case, kind):
    """Training under band masks (sliding window, packed documents; a (1,1,S,S) boolean mask): recognised as "row p
    sees first[p] .. p" and run through the differentiable kernel operators - the mask inside the scores kernel and the
    softmax kernel, zeros behind the post-softmax conv, the gradient with respect to the probabilities and the recomputed
    raw scores formed inside the band, the conv's input gradient zeroed outside it.  All seven gradients against autograd
    through the oracle given the mask tensor."""
    b, h, s, d, r1, s1, dtype = case
    print(f"mta module backward band mask {kind} {case}", flush=True)
    mod, params = _mta_pair(pkg, h, r1, s1, dtype, seed=381)
    mod.use_mask = True
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=382)
    visible = _band_masks(s)[kind][None, None]
    go = _rand((b, s, h, d), 383, dtype)
    want_out, want_in, want_w = _oracle_grads(q, k, v, params, go, mask=visible)
    stages = []
    mod._stage_hook = stages.append
    out, gin, gw = _module_grads(mod, q, k, v, go, mask=visible)
    assert "qk_conv" in stages and "conv_post" in stages and "pv" in stages, stages
    _check_all(dtype, out.cpu(), want_out, [g.cpu() for g in gin + gw], want_in + want_w)


def test_mta_module_backward_band_mask_without_the_kernels_takes_the_composite(pkg):
    """fp32 under a band mask in training: no in-place zeroing kernel, no lower-triangle products - the composite over the
    mask tensor runs, with the same answers."""
    print("mta module backward band mask fp32", flush=True)
    dtype = torch.float32
    b, h, s, d = 1, 4, 72, 64
    mod, params = _mta_pair(pkg, h, 3, 3, dtype, seed=391)
    mod.use_mask = True
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=392)
    visible = _band_masks(s)["window"][None, None]
    go = _rand((b, s, h, d), 393, dtype)
    want_out, want_in, want_w = _oracle_grads(q, k, v, params, go, mask=visible)
    out, gin, gw = _module_grads(mod, q, k, v, go, mask=visible)
    _check_all(dtype, out.cpu(), want_out, [g.cpu() for g in gin + gw], want_in + want_w)


@pytest.mark.parametrize("kind", ["window1024", "key_padding"])
def test_mta_module_backward_masks_benchmark_shape(pkg, kind):
    """The training step under mask tensors at the shape the benchmark times it (B1 H16 S4096 D128 fp16, 7x7 kernels,
    dense head weights), where the oracle on the host is out of reach: the route through the kernel operators against the
    module's own composite over the (B,H,S,S) mask tensor (torch's operators and the single-stage kernels; the route
    every mask took before it was recognised, pinned against the oracle at small sizes above), forward and all seven
    gradients, to the 16-bit bars."""
    print(f"mta module backward {kind} benchmark shape", flush=True)
    dtype = torch.float16
    b, h, s, d = 1, 16, 4096, 128
    mod, params = _mta_pair(pkg, h, 7, 7, dtype, seed=401)
    with torch.no_grad():   # a 7x7 post-softmax kernel as well
        w = O.seeded_conv_weight(h, 7, 7, 0.05, torch.float32, seed=402).to(dtype)
        mod.mta_conv_after_sm_triton = pkg.Conv2dTriton(h, (7, 7), causal=True).to(dtype).cuda()
        mod.mta_conv_after_sm_triton.weight.copy_(w)
    mod.use_mask = True
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=403)
    pos = torch.arange(s)
    lower = pos[None, :] <= pos[:, None]
    visible = (lower & (pos[None, :] > pos[:, None] - 1024)) if kind == "window1024" else (lower & (pos < 3000)[None, :])
    visible = visible[None, None]
    go = _rand((b, s, h, d), 404, dtype)
    stages = []
    mod._stage_hook = stages.append
    out, gin, gw = _module_grads(mod, q, k, v, go, mask=visible)
    assert "qk_conv" in stages, stages
    mod._stage_hook = None
    mod._structured_mask = lambda *a: (None, None)     # nothing recognised: the composite
    want_out, want_in, want_w = _module_grads(mod, q, k, v, go, mask=visible)
    _check_all(dtype, out.cpu(), want_out.cpu(), [g.cpu() for g in gin + gw], [g.cpu() for g in want_in + want_w])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mta_module_backward_non_causal_key_padding(pkg, dtype):
    """causal=False, use_mask=True, key padding of a batch, in training: the differentiable operators in their non-causal
    form with a key bias and zeroed K and V rows; all seven gradients against autograd through the oracle given the mask
    tensor."""
    print(f"mta module backward causal=False key padding {dtype}", flush=True)
    b, h, s, d = 2, 4, 136, 64
    mod, params = _mta_pair(pkg, h, 3, 5, dtype, seed=411, causal=False)
    mod.use_mask = True
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=412)
    keep = torch.arange(s)[None, :] < torch.tensor([136, 77])[:, None]
    visible = keep[:, None, None, :].expand(b, 1, s, s).contiguous()
    go = _rand((b, s, h, d), 413, dtype)
    want_out, want_in, want_w = _oracle_grads(q, k, v, params, go, mask=visible.expand(b, h, s, s))
    stages = []
    mod._stage_hook = stages.append
    out, gin, gw = _module_grads(mod, q, k, v, go, mask=visible)
    assert "pv" in stages and ("mix_softmax" in stages or "softmax" in stages), stages   # (the operator route's marks)
    _check_all(dtype, out.cpu(), want_out, [g.cpu() for g in gin + gw], want_in + want_w)
    real = keep[:, None, :, None]
    for name, g in (("xk", gin[1]), ("xv", gin[2])):
        assert not (g.cpu() * ~real).any(), f"grad {name} of a hidden key is not zero"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("causal", [True, False])
def test_mta_module_backward_arbitrary_mask_planes(pkg, causal, dtype):
    """Training under a mask of arbitrary content (random holes, a plane per head; boolean): the differentiable operators
    with the three mask steps as passes over uint8 visibility planes (forward in place; backward: the conv's input
    gradient and the gradient behind the post-softmax conv zeroed at the hidden positions).  All seven gradients against
    autograd through the oracle given the mask tensor."""
    print(f"mta module backward arbitrary mask causal={causal} {dtype}", flush=True)
    b, h, s, d = 2, 4, 136, 64
    mod, params = _mta_pair(pkg, h, 3, 5, dtype, seed=421, causal=causal)
    mod.use_mask = True
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=422)
    g = torch.Generator().manual_seed(423)
    visible = (torch.rand(1, h, s, s, generator=g) > 0.3) | torch.eye(s, dtype=torch.bool)
    if causal:
        visible &= torch.tril(torch.ones(s, s, dtype=torch.bool))
    go = _rand((b, s, h, d), 424, dtype)
    want_out, want_in, want_w = _oracle_grads(q, k, v, params, go, mask=visible.expand(b, h, s, s))
    stages = []
    mod._stage_hook = stages.append
    out, gin, gw = _module_grads(mod, q, k, v, go, mask=visible)
    assert stages.count("mask") == 3 and "pv" in stages, stages
    _check_all(dtype, out.cpu(), want_out, [g_.cpu() for g_ in gin + gw], want_in + want_w)
    # the same with an additive mask that holds finite values besides 0 and -inf (added ahead of the softmax)
    additive = torch.where(visible, 0.5 * torch.randn(1, h, s, s, generator=g), float("-inf")).to(dtype)
    want_out, want_in, want_w = _oracle_grads(q, k, v, params, go, mask=additive.expand(b, h, s, s))
    del stages[:]
    out, gin, gw = _module_grads(mod, q, k, v, go, mask=additive)
    assert stages.count("mask") == 3, stages
    _check_all(dtype, out.cpu(), want_out, [g_.cpu() for g_ in gin + gw], want_in + want_w)


@pytest.mark.parametrize("case", [(2, 4, 264, 64, 3, 3, torch.bfloat16), (2, 16, 520, 128, 6, 11, torch.float16)])
def test_mta_module_backward_left_padded_batch(pkg, case):
    """Training on a left-padded batch (a band mask whose padding rows see no key): the band route of the differentiable
    operators, the padding rows' probabilities cleared inside the softmax stage.  The reference's own gradients are NaN
    under such a mask (the softmax of an empty row), so: the forward against the oracle, gradients finite and zero for
    the padding, and all seven gradients against the mask-pass route (pinned against the oracle above) on the same mask."""
    b, h, s, d, r1, s1, dtype = case
    print(f"mta module backward left padding {case}", flush=True)
    mod, params = _mta_pair(pkg, h, r1, s1, dtype, seed=431)
    mod.use_mask = True
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=432)
    pad = torch.tensor([0, s // 4])
    keep = torch.arange(s)[None, :] >= pad[:, None]
    visible = keep[:, None, None, :] & torch.tril(torch.ones(s, s, dtype=torch.bool))[None, None]
    go = _rand((b, s, h, d), 433, dtype) * keep[:, :, None, None]
    want_out = O.mta_forward(q.float(), k.float(), v.float(), params[0].float().unsqueeze(1), params[1].float(),
                             params[2].float().unsqueeze(1), params[3].float(), mask=visible.expand(b, h, s, s))
    stages = []
    mod._stage_hook = stages.append
    out, gin, gw = _module_grads(mod, q, k, v, go, mask=visible)
    assert "mask" not in stages and "qk_conv" in stages and "pv" in stages, stages
    _close(out, want_out, dtype, "forward")
    assert not out[1, :int(pad[1])].any()
    for name, g_ in zip(_GRAD_NAMES, gin + gw):
        assert torch.isfinite(g_).all(), name
    for name, g_ in zip(("xq", "xk", "xv"), gin):
        assert not g_[1, :, :int(pad[1])].any(), f"the padding of {name} received a gradient"
    mod._band_training_supported = lambda *a: False      # the mask passes instead
    del stages[:]
    out2, gin2, gw2 = _module_grads(mod, q, k, v, go, mask=visible)
    assert stages.count("mask") >= 3, stages
    _check_all(dtype, out.cpu(), out2.cpu(), [g_.cpu() for g_ in gin + gw], [g_.cpu() for g_ in gin2 + gw2])


def test_mta_module_backward_key_mask_finite_values(pkg):
    """A 2-D additive key mask with finite values besides -inf (B = 1), in training: the values are added ahead of the
    softmax (mta_attention_triton.py:77), only -inf hides a key."""
    print("mta module backward additive key mask", flush=True)
    dtype = torch.bfloat16
    b, h, s, d = 1, 8, 264, 64
    mod, params = _mta_pair(pkg, h, 3, 5, dtype, seed=371)
    mod.use_mask = True
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=372)
    mask = torch.zeros(1, s)
    mask[0, 10:14] = float("-inf")
    mask[0, 100:120] = -1.5
    mask[0, 200] = 0.75
    go = _rand((b, s, h, d), 373, dtype)
    want_out, want_in, want_w = _oracle_grads(q, k, v, params, go, mask=mask.to(dtype))
    out, gin, gw = _module_grads(mod, q, k, v, go, mask=mask.to(dtype))
    _check_all(dtype, out.cpu(), want_out, [g.cpu() for g in gin + gw], want_in + want_w)


def test_mta_module_backward_with_dropout(pkg, monkeypatch):
    """Training mode with dropout 0.5 under a fixed seed.  The gradient with respect to the probabilities comes from the
    scores kernel, which writes nothing above the diagonal; the dropout's backward multiplies that buffer elementwise
    before the head mixing's gradient kernels read its lower triangle.  The result must be finite and agree with a run
    in which that gradient comes from the library GEMM (fully defined) - also when the memory the buffer is allocated
    from holds NaN."""
    import multitokenatention_triton_amd.mta_attention_triton as glue
    print("mta module backward dropout", flush=True)
    dtype = torch.bfloat16
    b, h, s, d = 1, 8, 264, 64
    mod, params = _mta_pair(pkg, h, 3, 3, dtype, seed=361)
    mod.dropout = 0.5
    mod.train()
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=362)
    go = _rand((b, s, h, d), 363, dtype)

    def run():
        torch.manual_seed(99)
        junk = [torch.full((b, h, s, s), float("nan"), dtype=dtype, device="cuda") for _ in range(4)]
        del junk   # the allocator hands these blocks to the next (B,H,S,S) tensors
        return _module_grads(mod, q, k, v, go)

    out1, gin1, gw1 = run()
    for t in [out1] + gin1 + gw1:
        assert torch.isfinite(t.float()).all()
    assert float((out1 == 0).float().mean()) < 0.5   # (dropout acts on the probabilities, not on the output)
    monkeypatch.setattr(glue, "_lower_scores", lambda a, c, first_visible=None: None)
    out2, gin2, gw2 = run()
    assert torch.equal(out1, out2)                   # same seed, same dropout mask
    for name, a_, c_ in zip(_GRAD_NAMES, gin1 + gw1, gin2 + gw2):
        _rel_norm(a_, c_.float(), dtype, f"grad {name}, kernel against GEMM for dP")
