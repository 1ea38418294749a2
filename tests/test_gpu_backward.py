"""GPU parity of the backward entry points (through the C ABI) against torch.autograd through the CPU oracle.

  mta_conv2d_bwd_input / _weight     vs oracle.depthwise_conv_grads   (convolution_2d_trit.py:143-295, 336-378)
  mta_headmix_bwd_input / _weight    vs oracle.head_linear_grads      (triton_linear_head.py:144-278, 322-370)
  MTAAttentionTriton(...).backward() vs autograd through oracle.mta_forward: the gradient checks of the
                                     reference's compare script (compare_mta_attention.py:123-162)

Tolerances.  fp32: rtol 1e-4, atol 1e-5 times the largest expected magnitude (weight gradients are sums over
up to 10^6 products, so the absolute floor scales with them).  bf16/fp16: inputs and the input gradient are
stored in 16 bits: 2e-2 times the largest expected magnitude; weight gradients are accumulated and returned
in fp32 from 16-bit inputs that the oracle sees as the same 16-bit values, so they keep rtol 1e-3.
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


def _mta_pair(pkg, h, r1, s1, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    params = [O.seeded_conv_weight(h, r1, s1, 0.1, torch.float32, seed=seed + 1),
              torch.eye(h) + 0.1 * torch.randn(h, h, generator=g),
              O.seeded_conv_weight(h, 3, 3, 0.1, torch.float32, seed=seed + 2),
              torch.eye(h) + 0.1 * torch.randn(h, h, generator=g)]
    params = [p.to(dtype) for p in params]
    cfg = pkg.MTAConfig(query_kernel_size=r1, key_kernel_size=s1)
    mod = pkg.MTAAttentionTriton(h, cfg, dropout=0.0, causal=True)
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
    for name, p_, wt in (("pre conv", mod.mta_conv_triton.weight, wl[0].grad), ("wpsm", mod.wpsm_triton.weight, wl[1].grad),
                         ("post conv", mod.mta_conv_after_sm_triton.weight, wl[2].grad),
                         ("wposm", mod.wposm_triton.weight, wl[3].grad)):
        assert p_.grad is not None and p_.grad.dtype == dtype
        if dtype == torch.float32:
            _close(p_.grad, wt, dtype, f"grad {name}")
        else:   # intermediate score tensors are stored in bf16 along the way: 16-bit tolerance on the sums
            _close(p_.grad, wt, dtype, f"grad {name}")


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
    for name, p_, wt in (("pre conv", mod.mta_conv_triton.weight, wl[0].grad), ("wpsm", mod.wpsm_triton.weight, wl[1].grad),
                         ("post conv", mod.mta_conv_after_sm_triton.weight, wl[2].grad),
                         ("wposm", mod.wposm_triton.weight, wl[3].grad)):
        _close(p_.grad, wt, dtype, f"grad {name}")


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
