"""GPU parity of the standalone operators (through the C ABI) against the CPU oracle.

Tolerances (written here once):
  fp32 I/O : rtol 1e-4, atol 1e-5
  bf16/fp16: atol 2e-2 plus one unit in the last place of the 16-bit format as rtol
             (2^-7 for bf16, 2^-10 for fp16) -- an op output of magnitude m cannot be
             pinned tighter than the oracle's own rounding of m.
Causal fill patterns (+0.0 / -inf above the diagonal) are compared bit-exactly.
"""
import pytest
import torch

from oracle import mta_oracle as O

pytestmark = pytest.mark.gpu

DT = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}


def tol(dtype):
    if dtype == torch.float32:
        return dict(rtol=1e-4, atol=1e-5)
    return dict(rtol=2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10, atol=2e-2)


def _randn(shape, seed, dtype, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return (std * torch.randn(*shape, generator=g)).to(dtype)


def _upper(p, q):
    return torch.triu(torch.ones(p, q, dtype=torch.bool), 1)


@pytest.fixture(scope="module")
def ops():
    from multitokenatention_triton_amd import ops as _ops
    return _ops


CONV_CASES = [
    # N, C, H(=W), R, S
    (1, 2, 1, 3, 3), (1, 1, 7, 1, 1), (2, 3, 37, 3, 5), (1, 2, 64, 6, 11), (1, 2, 130, 6, 11),
    (1, 1, 100, 4, 6), (1, 2, 96, 11, 15), (1, 1, 70, 2, 7), (1, 4, 256, 3, 5), (1, 1, 45, 32, 63),
    # widths divisible by 8: 16-bit inputs take the MFMA (Toeplitz) kernel
    (1, 2, 136, 6, 11), (2, 2, 520, 6, 11), (1, 1, 128, 7, 9), (1, 2, 264, 5, 7), (1, 1, 1032, 3, 3),
    (1, 3, 8, 6, 11), (1, 1, 392, 7, 7), (1, 2, 200, 5, 5),
    # several 256-key strips per row strip, ragged last one; 11x15 on the matrix cores
    (1, 2, 776, 6, 11), (1, 1, 128, 11, 15), (1, 2, 520, 11, 15), (3, 1, 264, 6, 11),
    # the largest kernel of the reference's published rows (77 x 77, benchmark_seq_len_results.jsonl:140-180) and the
    # largest the operator takes: general fp32-FMA kernel, staged tile beyond 64 KB of LDS
    (1, 1, 96, 77, 77), (1, 1, 40, 80, 95),
]


@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("case", CONV_CASES)
def test_conv_parity(ops, case, causal, dt):
    n, c, s, r, sk = case
    dtype = DT[dt]
    print(f"conv case={case} causal={causal} dt={dt}", flush=True)
    x = _randn((n, c, s, s), 1, dtype)
    if causal:
        x = torch.tril(x)
    w = _randn((c, r, sk), 2, dtype, 0.2)
    want = O.depthwise_conv(x.float(), w.float(), causal)
    want_rounded = want.to(dtype)
    got = ops.conv2d_causal(x.cuda(), w.cuda(), causal).cpu()
    assert got.dtype == dtype and got.shape == x.shape
    torch.testing.assert_close(got.float(), want_rounded.float(), **tol(dtype))
    if causal:
        up = _upper(s, s)
        assert (got[..., up] == 0).all() and not torch.signbit(got[..., up]).any()


@pytest.mark.parametrize("wdt", ["f32", "bf16"])
def test_conv_weight_dtype_and_scale(ops, wdt):
    x = torch.tril(_randn((1, 2, 80, 80), 3, torch.bfloat16, 8.0))
    w = _randn((2, 6, 11), 4, DT[wdt], 0.05)
    scale = float(torch.rsqrt(torch.tensor(128.0)))
    xs = x * torch.rsqrt(torch.tensor(128))          # bf16 result, as the reference computes it
    want = O.depthwise_conv(xs.float(), w.float(), True).to(torch.bfloat16)
    got = ops.conv2d_causal(x.cuda(), w.cuda(), True, in_scale=scale).cpu()
    torch.testing.assert_close(got.float(), want.float(), **tol(torch.bfloat16))


def test_conv_identity_tap_bit_exact(ops):
    for dtype in (torch.float32, torch.bfloat16):
        x = _randn((2, 3, 77, 77), 5, dtype)
        w = O.identity_conv_kernel(3, 6, 11, dtype)
        got = ops.conv2d_causal(x.cuda(), w.cuda(), True).cpu()
        assert torch.equal(got, torch.tril(x) + 0.0)


def test_conv_delta_is_shift(ops):
    x = torch.tril(_randn((1, 1, 50, 50), 6, torch.float32))
    for (i, j) in [(0, 0), (2, 4), (5, 10), (3, 5)]:
        w = torch.zeros(1, 6, 11)
        w[0, i, j] = 1.0
        got = ops.conv2d_causal(x.cuda(), w.cuda(), True).cpu()
        assert torch.equal(got, O.depthwise_conv(x, w, True))


MFMA_KERNEL_SIZES = [(3, 3), (3, 5), (5, 5), (5, 7), (6, 11), (7, 7), (7, 9), (11, 15)]


@pytest.mark.parametrize("plane", [(32, 128), (32, 256), (64, 512)])
@pytest.mark.parametrize("rs", MFMA_KERNEL_SIZES)
def test_conv_channel_changes_on_every_strip(ops, rs, plane):
    """Every kernel size with a matrix-core instance, forward and input gradient, on planes that hold a single strip
    (32 rows x 256 keys; half a strip; four strips) each: consecutive work items of a workgroup then belong to different
    channels all the time, so the kernel rows fetched one strip ahead are consumed on every iteration, with odd tap counts
    (3x3, 5x5, ... : every other channel's kernel starts in the middle of a 32-bit word).  Channels get very different
    weights so that a kernel row applied to the wrong strip cannot pass."""
    r, s = rs
    print(f"conv channel change rs={rs} plane={plane}", flush=True)
    dtype = torch.bfloat16
    n, c = 3, 24
    h, wd = plane
    x = _randn((n, c, h, wd), 31, dtype)
    w = (_randn((c, r, s), 32, torch.float32, 0.2) * (1.0 + torch.arange(c)[:, None, None])).to(dtype)
    for causal in (False, True):
        want = O.depthwise_conv(x.float(), w.float(), causal).to(dtype)
        got = ops.conv2d_causal(x.cuda(), w.cuda(), causal).cpu()
        torch.testing.assert_close(got.float(), want.float(), rtol=2.0 ** -7, atol=2e-2 * c)
        dy = _randn((n, c, h, wd), 33, dtype)
        want_dx, _ = O.depthwise_conv_grads(x.float(), w.float(), causal, dy.float())
        got_dx = ops.conv2d_bwd_input(dy.cuda(), w.cuda(), causal).cpu()
        torch.testing.assert_close(got_dx.float(), want_dx.to(dtype).float(), rtol=2.0 ** -7, atol=2e-2 * c)


def test_conv_non_finite_input_stays_local(ops):
    """The matrix-core kernel multiplies a 32-key window by a zero-padded tap matrix, so one inf at an attended
    position turns every output of its 16-key block (and of the neighbouring block whose window holds it), in the R
    rows below it, into NaN -- a wider footprint than the R x S taps of the fp32-FMA kernel.  Outputs further away
    must be what they are without the inf, and the true footprint must be non-finite in both kernels."""
    print("conv inf input", flush=True)
    r, s = 6, 11
    w = _randn((1, r, s), 41, torch.float32, 0.2).abs() + 0.05      # no zero taps: the true footprint is all non-finite
    x = torch.tril(_randn((1, 1, 256, 256), 42, torch.float32))
    clean16 = ops.conv2d_causal(x.bfloat16().cuda(), w.bfloat16().cuda(), True).cpu().float()
    clean32 = ops.conv2d_causal(x.cuda(), w.cuda(), True).cpu()
    p0, q0 = 100, 40
    x[0, 0, p0, q0] = float("inf")
    got16 = ops.conv2d_causal(x.bfloat16().cuda(), w.bfloat16().cuda(), True).cpu().float()   # matrix cores
    got32 = ops.conv2d_causal(x.cuda(), w.cuda(), True).cpu()                                 # fp32 FMAs
    foot = torch.zeros(256, 256, dtype=torch.bool)
    foot[p0:p0 + r, q0 - (s - 1) // 2:q0 + (s - 1) // 2 + 1] = True
    assert not torch.isfinite(got32[0, 0][foot]).any() and not torch.isfinite(got16[0, 0][foot]).any()
    assert torch.equal(got32[0, 0][~foot], clean32[0, 0][~foot])
    wide = torch.zeros(256, 256, dtype=torch.bool)
    wide[p0:p0 + r, q0 - 32:q0 + 32] = True
    assert torch.equal(got16[0, 0][~wide], clean16[0, 0][~wide])


HM_CASES = [
    # N, C, P, Q, group (None = dense)
    (1, 4, 9, 9, None), (2, 4, 64, 64, 2), (1, 8, 40, 40, 4), (1, 6, 33, 33, None), (1, 6, 24, 24, 3),
    (1, 16, 48, 48, None), (1, 32, 16, 16, 4), (1, 32, 24, 24, None), (2, 2, 300, 300, 1), (1, 4, 5, 2056, 2),
    # 32 heads mixed densely (matrix-core kernel for 16-bit data): several wavefronts and workgroups per row, ragged
    # last wavefront, rows longer and shorter than the key range, two groups of 32
    (1, 32, 300, 296, None), (1, 32, 40, 1160, None), (2, 64, 136, 136, 32), (1, 32, 600, 64, None),
    # 64 and 128 heads mixed densely (the head counts of the reference's own benchmark rows,
    # benchmark_seq_len_results.jsonl:198-213): contraction over 2 / 4 blocks of 32 input heads, two wavefronts per key
    # chunk for 128 heads; ragged last chunk; two groups of 64
    (1, 64, 200, 200, None), (1, 128, 136, 136, None), (1, 128, 24, 520, None), (1, 128, 264, 264, 64), (2, 64, 40, 1032, None),
]


@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("causal,fill", [(True, 0.0), (True, float("-inf")), (False, 0.0)])
@pytest.mark.parametrize("case", HM_CASES)
def test_headmix_parity(ops, case, causal, fill, dt):
    n, c, p, q, group = case
    dtype = DT[dt]
    print(f"headmix case={case} causal={causal} fill={fill} dt={dt}", flush=True)
    x = _randn((n, c, p, q), 7, dtype)
    g = torch.Generator().manual_seed(8)
    if group:
        w = O.block_diag_head_weight(c, group, 0.1, g, dtype)
    else:
        w = (torch.eye(c) + 0.1 * torch.randn(c, c, generator=g)).to(dtype)
    want = O.head_linear(x.float(), w.float(), causal, fill).to(dtype)
    got = ops.headmix(x.cuda(), w.cuda(), causal, fill, group_size=group).cpu()
    if causal:
        up = _upper(p, q)
        if fill == 0.0:
            assert (got[..., up] == 0).all() and not torch.signbit(got[..., up]).any()
        else:
            assert torch.isneginf(got[..., up]).all()
        low = ~up
        torch.testing.assert_close(got[..., low].float(), want[..., low].float(), **tol(dtype))
    else:
        torch.testing.assert_close(got.float(), want.float(), **tol(dtype))
    if group:  # the group hint must not change the result of the dense contraction
        dense = ops.headmix(x.cuda(), w.cuda(), causal, fill, group_size=None).cpu()
        torch.testing.assert_close(dense.float().nan_to_num(neginf=-1e30), got.float().nan_to_num(neginf=-1e30),
                                   **tol(dtype))


def test_headmix_identity_and_permutation_bit_exact(ops):
    x = _randn((1, 4, 31, 31), 9, torch.bfloat16)
    got = ops.headmix(x.cuda(), torch.eye(4).cuda(), True, 0.0).cpu()
    assert torch.equal(got, torch.tril(x) + 0.0)
    perm = torch.tensor([2, 0, 3, 1])
    wp = torch.zeros(4, 4)
    wp[torch.arange(4), perm] = 1.0
    got = ops.headmix(x.cuda(), wp.cuda(), True, 0.0).cpu()
    assert torch.equal(got, torch.tril(x[:, perm]) + 0.0)


@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("case", [(1, 2, 384, 6, 11), (2, 3, 200, 3, 3), (1, 2, 1024, 7, 7), (1, 1, 72, 11, 15)])
def test_conv_tril_leaves_the_upper_triangle_alone(ops, case, dt):
    """fill_upper=False: the lower triangle (diagonal included) is bit for bit what the filling call writes; above it
    the output holds either what was there (sentinel) or +0."""
    n, c, s, r, sk = case
    dtype = DT[dt]
    print(f"conv tril case={case} dt={dt}", flush=True)
    x = torch.tril(_randn((n, c, s, s), 21, dtype)).cuda()
    w = _randn((c, r, sk), 22, dtype, 0.2).cuda()
    full = ops.conv2d_causal(x, w, True)
    out = torch.full_like(x, 7.0)
    got = ops.conv2d_causal(x, w, True, out=out, fill_upper=False)
    low = ~_upper(s, s).cuda()
    assert torch.equal(got[..., low], full[..., low])
    up = got[..., ~low].float()
    assert ((up == 7.0) | (up == 0)).all()
    if dtype != torch.float32 and s % 128 == 0 and (r, sk) != (11, 15):   # the matrix-core kernel: blocks wholly above stay untouched
        assert (got[..., 0, s - 128:].float() == 7.0).all()


@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("case", [(1, 8, 300, 4), (2, 4, 2304, 2), (1, 32, 520, 0), (1, 16, 264, 0), (1, 6, 100, 3)])
def test_headmix_tril_leaves_the_upper_triangle_alone(ops, case, dt):
    n, c, s, group = case
    dtype = DT[dt]
    print(f"headmix tril case={case} dt={dt}", flush=True)
    x = _randn((n, c, s, s), 23, dtype).cuda()
    g = torch.Generator().manual_seed(24)
    w = (O.block_diag_head_weight(c, group, 0.1, g, dtype) if group else
         (torch.eye(c) + 0.1 * torch.randn(c, c, generator=g)).to(dtype)).cuda()
    full = ops.headmix(x, w, True, 0.0, group_size=group or None)
    out = torch.full_like(x, 7.0)
    got = ops.headmix(x, w, True, 0.0, group_size=group or None, out=out, fill_upper=False)
    low = ~_upper(s, s).cuda()
    assert torch.equal(got[..., low], full[..., low])
    up = got[..., ~low].float()
    assert ((up == 7.0) | (up == 0)).all()
    if s >= 2048:   # whole chunks of a row above the diagonal are never touched
        assert (got[..., 0, s - 64:].float() == 7.0).all()


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("case", [(1, 2, 384, 6, 11), (2, 2, 264, 7, 7), (1, 3, 100, 3, 3)])
def test_lower_only_mode_of_the_other_conv_and_headmix_entries(ops, case, dt):
    """`causal` = MTA_CAUSAL_LOWER_ONLY in mta_conv2d_scaled_fwd, mta_conv2d_bwd_input and mta_headmix_bwd_input: on and
    below the diagonal bit for bit the filling call's result, above it the buffer's old content (sentinel) or +0."""
    n, c, s, r, sk = case
    dtype = DT[dt]
    print(f"lower-only case={case} dt={dt}", flush=True)
    x = torch.tril(_randn((n, c, s, s), 31, dtype)).cuda()
    w = _randn((c, r, sk), 32, dtype, 0.2).cuda()
    g = torch.Generator().manual_seed(33)
    wm = (torch.eye(c) + 0.1 * torch.randn(c, c, generator=g)).to(dtype).cuda()
    low = ~_upper(s, s).cuda()
    sent = lambda: torch.full_like(x, 7.0)
    pairs = [
        (ops.conv2d_causal(x, w, True, in_scale=0.125), ops.conv2d_causal(x, w, True, in_scale=0.125, out=sent(), fill_upper=False)),
        (ops.conv2d_bwd_input(x, w, True), ops.conv2d_bwd_input(x, w, True, fill_upper=False, out=sent())),
        (ops.headmix_bwd_input(x, wm, True), ops.headmix_bwd_input(x, wm, True, fill_upper=False, out=sent())),
    ]
    for full, got in pairs:
        assert torch.equal(got[..., low], full[..., low])
        up = got[..., ~low].float()
        assert ((up == 7.0) | (up == 0)).all()
    if dtype != torch.float32 and s % 128 == 0:   # matrix-core conv kernels: blocks wholly above the diagonal stay untouched
        for _, got in pairs[:2]:
            assert (got[..., 0, s - 128:].float() == 7.0).all()


MS_CASES = [
    # N, C, P(=Q), group, use_w1, use_w2
    (1, 4, 64, 2, True, True), (2, 4, 100, 4, True, False), (1, 8, 257, 4, False, True), (1, 2, 33, 1, False, False),
    (1, 8, 2048, 4, True, True), (1, 3, 50, 3, True, True), (1, 8, 72, 8, True, True), (1, 4, 4096, 4, True, True),
    # packed-arithmetic kernel (16-bit data): one weight only, several passes with few heads, rows that end inside
    # a wavefront's pass / exactly on its boundary (2560 = 5 x 512), rectangular
    (1, 4, 3000, 4, False, True), (1, 4, 2560, 4, True, False), (1, 2, 6000, 2, True, True), (1, 8, 520, 8, False, True),
    # groups of 16 heads (16-bit data: both mixes on the matrix cores): one and both weights, two groups, rows that end
    # inside a tile of 128 keys / on its boundary, the longest row the kernel takes
    (1, 16, 200, 16, True, False), (2, 16, 264, 16, True, True), (1, 32, 136, 16, False, True), (1, 16, 2048, 16, True, True),
    (1, 16, 4096, 16, True, False),
    # lists of rows per workgroup with several steps each: two batch entries and two groups, rows of all three kinds
    # (4, 8, 16 wavefronts); rows that end inside a tile with the second weight only
    (2, 32, 2304, 16, True, True), (1, 16, 3000, 16, False, True),
    # no weights, rows of up to 2048 keys (16-bit data: a wavefront per row): rows that end inside a lane's vector, the
    # longest rows, several planes and batch entries; 2056 keys: back to a workgroup per row
    (2, 3, 520, 1, False, False), (1, 2, 2048, 1, False, False), (1, 4, 72, 1, False, False), (1, 2, 2056, 1, False, False),
]


@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("case", MS_CASES)
def test_mix_softmax_mix_parity(ops, case, causal, dt):
    n, c, s, group, use1, use2 = case
    dtype = DT[dt]
    if dt == "f32" and n * c * s * s > (1 << 27):
        pytest.skip("a GB of fp32 scores: the 16-bit runs cover this shape")
    print(f"mix_softmax_mix case={case} causal={causal} dt={dt}", flush=True)
    x = _randn((n, c, s, s), 10, dtype, 2.0)
    g = torch.Generator().manual_seed(11)
    w1 = O.block_diag_head_weight(c, group, 0.1, g, dtype) if use1 else None
    w2 = O.block_diag_head_weight(c, group, 0.1, g, dtype) if use2 else None
    s2 = O.head_linear(x, w1, causal, float("-inf")) if use1 else (
        x.masked_fill(_upper(s, s), float("-inf")) if causal else x)
    p0 = torch.softmax(s2.float(), -1).to(dtype)
    want = O.head_linear(p0, w2, causal, 0.0) if use2 else p0
    got = ops.headmix_softmax(x.cuda(), w1.cuda() if use1 else None, w2.cuda() if use2 else None, causal,
                              group_size=group).cpu()
    if causal:
        up = _upper(s, s)
        assert (got[..., up] == 0).all() and not torch.signbit(got[..., up]).any()
    t = tol(dtype)
    torch.testing.assert_close(got.float(), want.float(), rtol=t["rtol"] * 2, atol=2e-3 if dtype != torch.float32 else 1e-6)


@pytest.mark.parametrize("dt", ["bf16", "f16"])
@pytest.mark.parametrize("case", [(1, 16, 2560, True, True), (2, 16, 1160, True, False), (1, 32, 4096, False, True)])
def test_mix_softmax_mix_dense16_leaves_the_upper_triangle_alone(ops, case, dt):
    """Groups of 16 heads with fill_upper=False: on and below the diagonal bit for bit the filling call's result, above it
    the buffer's old content (or +0 inside the tile the diagonal crosses); NaN above the diagonal of the input is
    never read."""
    n, c, s, use1, use2 = case
    dtype = DT[dt]
    print(f"mix_softmax_mix dense16 lower-only case={case} dt={dt}", flush=True)
    x = _gpu_randn((n, c, s, s), 41, dtype, 2.0)
    g = torch.Generator().manual_seed(42)
    w1 = O.block_diag_head_weight(c, 16, 0.1, g, dtype).cuda() if use1 else None
    w2 = O.block_diag_head_weight(c, 16, 0.1, g, dtype).cuda() if use2 else None
    full = ops.headmix_softmax(x, w1, w2, True, group_size=16)
    up = _upper(s, s).cuda()
    got = ops.headmix_softmax(x.masked_fill(up, float("nan")), w1, w2, True, group_size=16, out=torch.full_like(x, 7.0),
                              fill_upper=False)
    assert torch.equal(got[..., ~up], full[..., ~up])
    above = got[..., up].float()
    assert ((above == 7.0) | (above == 0)).all()
    assert (got[..., 0, 128:].float() == 7.0).all()


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("case", [(1, 4, 64, 2, True, True), (2, 4, 100, 4, True, False), (1, 8, 257, 4, False, True),
                                  (2, 8, 2048, 4, True, True), (1, 8, 72, 8, True, True), (1, 2, 33, 1, False, False),
                                  (1, 4, 4096, 4, False, True),
                                  # groups of 16 heads (the matrix-core kernel's row lists, the bias row in LDS)
                                  (2, 16, 264, 16, True, True), (1, 32, 1160, 16, True, False), (1, 16, 2304, 16, False, True)])
def test_mix_softmax_mix_key_bias(ops, case, dt):
    """`scores = scores + mask` of mta_attention_triton.py:77-78 for a mask that is the causal rule plus one value per
    key: hidden keys (-inf) get probability 0, finite values are added in the I/O dtype."""
    n, c, s, group, use1, use2 = case
    dtype = DT[dt]
    print(f"mix_softmax_mix key bias case={case} dt={dt}", flush=True)
    x = _randn((n, c, s, s), 12, dtype, 2.0)
    g = torch.Generator().manual_seed(13)
    w1 = O.block_diag_head_weight(c, group, 0.1, g, dtype) if use1 else None
    w2 = O.block_diag_head_weight(c, group, 0.1, g, dtype) if use2 else None
    bias = torch.randn(n, s, generator=g).to(dtype).float()        # finite part, representable in the I/O dtype
    bias[torch.rand(n, s, generator=g) < 0.3] = float("-inf")
    bias[:, 0] = 0.0                                                # key 0 stays visible: no row is fully hidden
    s2 = O.head_linear(x, w1, True, float("-inf")) if use1 else x.masked_fill(_upper(s, s), float("-inf"))
    s3 = s2 + bias[:, None, None, :].to(dtype)                       # the reference's add, in the I/O dtype
    p0 = torch.softmax(s3.float(), -1).to(dtype)
    want = O.head_linear(p0, w2, True, 0.0) if use2 else p0
    got = ops.headmix_softmax(x.cuda(), w1.cuda() if use1 else None, w2.cuda() if use2 else None, True,
                              group_size=group, key_bias=bias.cuda()).cpu()
    up = _upper(s, s)
    assert (got[..., up] == 0).all() and not torch.signbit(got[..., up]).any()
    if not use2:
        hidden = torch.isinf(bias)[:, None, None, :].expand_as(got)
        assert (got[hidden] == 0).all()
    t = tol(dtype)
    torch.testing.assert_close(got.float(), want.float(), rtol=t["rtol"] * 2, atol=2e-3 if dtype != torch.float32 else 1e-6)
    with pytest.raises(ValueError):
        ops.headmix_softmax(x.cuda(), None, None, True, key_bias=bias.cuda().half())


CH_CASES = [
    # N, C, H(=W), R, S, group (None = dense)
    (1, 4, 64, 3, 3, 2), (2, 4, 100, 3, 3, 4), (1, 8, 264, 3, 3, 4), (1, 16, 136, 3, 3, None), (1, 16, 200, 7, 7, None),
    (1, 8, 72, 5, 7, 8), (1, 2, 33, 3, 5, 1), (1, 6, 50, 2, 2, 2), (1, 32, 96, 3, 3, 16),
    # dense groups of 16 heads at 16-bit dtypes: conv and mixing on the matrix cores, several items per workgroup
    (2, 32, 328, 7, 7, 16), (1, 16, 520, 5, 5, None), (1, 16, 776, 3, 3, None),
]


@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("case", CH_CASES)
def test_conv_headmix_parity(ops, case, causal, dt):
    """mta_conv_after_sm_triton -> wposm_triton (mta_attention_triton.py:81-85) as one kernel, against the oracle's
    conv (rounded to the I/O dtype, as the unfused pipeline stores it) followed by its head mixing."""
    n, c, s, r, sk, group = case
    dtype = DT[dt]
    print(f"conv_headmix case={case} causal={causal} dt={dt}", flush=True)
    g = torch.Generator().manual_seed(21)
    x = torch.softmax(_randn((n, c, s, s), 20, torch.float32, 2.0).masked_fill(_upper(s, s) if causal else torch.zeros(s, s, dtype=torch.bool), float("-inf")), -1).to(dtype)
    wc = _randn((c, r, sk), 22, dtype, 0.3)
    wm = O.block_diag_head_weight(c, group or c, 0.3, g, dtype)
    t = O.depthwise_conv(x.float(), wc.float(), causal).to(dtype)
    want = O.head_linear(t, wm, causal, 0.0)
    for fill in (True, False):
        got = ops.conv2d_headmix(x.cuda(), wc.cuda(), wm.cuda(), causal, group_size=group, fill_upper=fill)
        assert got is not None and got.dtype == dtype
        got = got.cpu()
        if causal:
            up = _upper(s, s)
            if fill:
                assert (got[..., up] == 0).all() and not torch.signbit(got[..., up]).any()
            got = torch.tril(got)
        torch.testing.assert_close(got.float(), want.float(), **tol(dtype))
    # mix weights of another dtype than the data take the plain multiply-add path
    if dtype != torch.float32:
        got = ops.conv2d_headmix(x.cuda(), wc.cuda(), wm.float().cuda(), causal, group_size=group).cpu()
        torch.testing.assert_close(got.float(), want.float(), **tol(dtype))


@pytest.mark.parametrize("dt", ["bf16", "f16"])
@pytest.mark.parametrize("ks", [(3, 3), (7, 7)])
def test_conv_headmix_dense16_equals_the_two_operators(ops, ks, dt):
    """Dense groups of 16 heads at a benchmark-sized plane (B1 H16 S2048): the one-pass kernel against conv followed by
    head mixing - the same products in the same order, so bit for bit on and below the diagonal - with the input above
    the diagonal poisoned (it must never be read), in both fill modes and without the causal rule."""
    dtype = DT[dt]
    s, c = 2048, 16
    print(f"conv_headmix dense16 ks={ks} dt={dt}", flush=True)
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.softmax(torch.randn(1, c, s, s, device="cuda", generator=g) * 2 +
                      torch.triu(torch.full((s, s), float("-inf"), device="cuda"), 1), -1).to(dtype)
    wc = (torch.randn(c, *ks, device="cuda", generator=g) * 0.3).to(dtype)
    wm = (torch.randn(c, c, device="cuda", generator=g) * 0.3).to(dtype)
    want = ops.headmix(ops.conv2d_causal(x, wc, True), wm, True, 0.0)
    poisoned = x.masked_fill(torch.triu(torch.ones(s, s, dtype=torch.bool, device="cuda"), 1), float("nan"))
    for fill in (True, False):
        got = ops.conv2d_headmix(poisoned, wc, wm, True, fill_upper=fill)
        assert got is not None
        if fill:
            assert torch.equal(got, want)
        else:
            assert torch.equal(torch.tril(got), torch.tril(want))
    want = ops.headmix(ops.conv2d_causal(x, wc, False), wm, False, 0.0)
    assert torch.equal(ops.conv2d_headmix(x, wc, wm, False), want)


def test_conv_headmix_unsupported_group(ops):
    x = torch.zeros(1, 12, 16, 16, device="cuda")
    assert ops.conv2d_headmix(x, torch.zeros(12, 3, 3, device="cuda"), torch.eye(12, device="cuda"), True) is None
    assert ops.conv2d_headmix(x, torch.zeros(12, 3, 3, device="cuda"), torch.eye(12, device="cuda"), True,
                              group_size=4) is not None


def test_error_codes(ops):
    x = torch.zeros(1, 2, 8, 8, device="cuda")
    with pytest.raises(ValueError, match="kernel size"):
        ops.conv2d_causal(x, torch.zeros(2, 81, 3, device="cuda"), True)     # (up to 80 x 95)
    with pytest.raises(ValueError, match="group"):
        ops.headmix(torch.zeros(1, 6, 8, 8, device="cuda"), torch.eye(6).cuda(), True, 0.0, group_size=4)
    with pytest.raises(AssertionError):
        ops.conv2d_causal(x, torch.zeros(3, 3, 3, device="cuda"), True)
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.conv2d_causal(x.cpu(), torch.zeros(2, 3, 3), True)


# ---- the benchmark configurations at their full sizes ---------------------------------------------------------
# Inputs are drawn on the GPU (a CPU generator needs most of a minute for 2.7e8 values).  Every channel / mixing
# group is independent of the others, so the oracle is run on a slice (what the CPU finishes in seconds) and the
# rest of the tensor is covered by properties that hold at any size: the identity kernel / permutation weight
# reproduces the input bit for bit, the causal fill pattern is exact everywhere, rows of probabilities sum to 1.

def _gpu_randn(shape, seed, dtype, std=1.0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (std * torch.randn(*shape, generator=g, device="cuda")).to(dtype)


def test_conv_full_size(ops):
    """BASELINE config 2: (2,16,2048,2048) bf16, 6x11 causal."""
    print("conv full size", flush=True)
    n, c, s, dtype = 2, 16, 2048, torch.bfloat16
    x = torch.tril(_gpu_randn((n, c, s, s), 20, dtype))
    w = _randn((c, 6, 11), 21, dtype, 0.2)
    got = ops.conv2d_causal(x, w.cuda(), True)
    up = _upper(s, s).cuda()
    assert (got[..., up] == 0).all() and not torch.signbit(got[..., up]).any()
    bi, c0 = 1, 5  # oracle on two channels of the second batch element
    want = O.depthwise_conv(x[bi:bi + 1, c0:c0 + 2].cpu().float(), w[c0:c0 + 2].float(), True).to(dtype)
    torch.testing.assert_close(got[bi:bi + 1, c0:c0 + 2].cpu().float(), want.float(), **tol(dtype))
    ident = ops.conv2d_causal(x, O.identity_conv_kernel(c, 6, 11, dtype).cuda(), True)
    assert torch.equal(ident, x + 0.0)


def test_headmix_full_size(ops):
    """BASELINE config 3: (2,32,2048,2048) bf16, groups of 4, and the dense 32x32 weight on the same tensor."""
    print("headmix full size", flush=True)
    n, c, s, dtype = 2, 32, 2048, torch.bfloat16
    x = _gpu_randn((n, c, s, s), 22, dtype)
    g = torch.Generator().manual_seed(23)
    up = _upper(s, s).cuda()
    low = ~_upper(s, s)
    for group in (4, None):
        w = O.block_diag_head_weight(c, 4, 0.1, g, dtype) if group else (
            torch.eye(c) + 0.1 * torch.randn(c, c, generator=g)).to(dtype)
        got = ops.headmix(x, w.cuda(), True, 0.0, group_size=group)
        assert (got[..., up] == 0).all() and not torch.signbit(got[..., up]).any()
        # oracle on the second batch element: one mixing group, or all 32 heads of the first 256 query rows
        bi = 1
        if group:
            sl, rows = slice(8, 12), slice(0, s)
            want = O.head_linear(x[bi:bi + 1, sl].cpu().float(), w[sl, sl].float(), True, 0.0).to(dtype)
        else:
            sl, rows = slice(0, c), slice(0, 256)
            want = O.head_linear(x[bi:bi + 1, :, rows].cpu().float(), w.float(), True, 0.0).to(dtype)
        sub = got[bi:bi + 1, sl, rows].cpu()
        m = low[rows]
        torch.testing.assert_close(sub[..., m].float(), want[..., m].float(), **tol(dtype))
    perm = torch.arange(c).roll(5)
    wp = torch.zeros(c, c, dtype=dtype)
    wp[torch.arange(c), perm] = 1.0
    got = ops.headmix(x, wp.cuda(), True, 0.0)  # dense weight that only permutes the heads: bit exact
    assert torch.equal(got, torch.tril(x[:, perm]) + 0.0)


def test_mix_softmax_mix_full_size(ops):
    """The score pass of BASELINE config 4: (2,16,4096,4096) bf16, groups of 4, both mixes."""
    print("mix_softmax_mix full size", flush=True)
    n, c, s, grp, dtype = 2, 16, 4096, 4, torch.bfloat16
    x = _gpu_randn((n, c, s, s), 24, dtype, 2.0)
    g = torch.Generator().manual_seed(25)
    w1 = O.block_diag_head_weight(c, grp, 0.1, g, dtype)
    w2 = O.block_diag_head_weight(c, grp, 0.1, g, dtype)
    got = ops.headmix_softmax(x, w1.cuda(), w2.cuda(), True, group_size=grp)
    # rows of probabilities sum to 1 before the second mix, so rows of the output sum to the row sums of w2
    rs = got.float().tril().sum(-1)
    want_rs = w2.float().sum(1)[None, :, None].cuda().expand_as(rs)
    torch.testing.assert_close(rs, want_rs, rtol=0.0, atol=3e-2)
    bi, sl = 1, slice(4, 8)
    xs = x[bi:bi + 1, sl].cpu()
    s2 = O.head_linear(xs, w1[sl, sl], True, float("-inf"))
    p0 = torch.softmax(s2.float(), -1).to(dtype)
    want = O.head_linear(p0, w2[sl, sl], True, 0.0)
    sub = got[bi:bi + 1, sl].cpu()
    up = _upper(s, s)
    assert (sub[..., up] == 0).all()
    torch.testing.assert_close(sub.float(), want.float(), rtol=2.0 ** -6, atol=2e-3)
