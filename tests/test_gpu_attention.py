"""GPU parity of the two attention entry points against the CPU oracle.

  MTAAttentionTriton.forward      vs oracle.mta_forward            (mta_attention_pytorch.py:58-83)
  TritonConvAttention.forward     vs oracle.conv_attention_forward (conv_attention_pytorch.py:33-71)

Tolerances: fp32 rtol 1e-4 / atol 1e-5; bf16 and fp16 atol 2e-2 (outputs are convex
combinations of N(0,1) values, so |out| is O(1) and no rtol is added).
"""
import pytest
import torch
import torch.nn.functional as F

from oracle import mta_oracle as O

pytestmark = pytest.mark.gpu


def tol(dtype):
    return dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=0.0, atol=2e-2)


@pytest.fixture(scope="module")
def pkg():
    import multitokenatention_triton_amd as m
    return m


def _mta_module(pkg, h, r1, s1, r2, s2, w_pre, wpsm, w_post, wposm, dtype, causal=True, use_mask=False,
                structure="infer"):
    """Inference-mode module on the GPU (parameters do not require grad, so forward takes the fused route).
    structure: "infer" = look at the weights once, "dense" = assume nothing, "probe" = look on every call."""
    cfg = pkg.MTAConfig(query_kernel_size=r1, key_kernel_size=s1, after_sm_query_kernel_size=r2,
                        after_sm_key_kernel_size=s2)
    mod = pkg.MTAAttentionTriton(h, cfg, dropout=0.0, causal=causal, use_mask=use_mask)
    with torch.no_grad():
        mod.mta_conv_triton.weight.copy_(w_pre)
        mod.wpsm_triton.weight.copy_(wpsm)
        mod.mta_conv_after_sm_triton.weight.copy_(w_post)
        mod.wposm_triton.weight.copy_(wposm)
    mod = mod.to(dtype).cuda().eval().requires_grad_(False)
    if structure == "infer":
        mod.infer_weight_structure()
    elif structure == "probe":
        mod.weight_structure = "probe"
    else:
        assert structure == "dense" and mod.weight_structure == "dense"
    return mod


def _config_like(h, group, r1, s1, std, dtype, post="identity", seed=123):
    g = torch.Generator().manual_seed(seed + 2)
    w_pre = O.seeded_conv_weight(h, r1, s1, std, torch.float32, seed=seed + 1)
    wpsm = O.block_diag_head_weight(h, group, 0.1, g)
    wposm = O.block_diag_head_weight(h, group, 0.1, g)
    if post == "identity":
        w_post = O.identity_conv_kernel(h, 3, 3)
    else:
        w_post = O.seeded_conv_weight(h, 3, 3, 0.05, torch.float32, seed=seed + 3)
    return [t.to(dtype) for t in (w_pre, wpsm, w_post, wposm)]


def _oracle_mta(q, k, v, params):
    w_pre, wpsm, w_post, wposm = params
    return O.mta_forward(q, k, v, w_pre.unsqueeze(1), wpsm, w_post.unsqueeze(1), wposm)


def test_mta_config1_fp32(pkg):
    """BASELINE config 1: B1 H4 S256 D64 fp32, 3x5 conv + identity tap, head-mix groups of 2."""
    print("mta config1 fp32", flush=True)
    q, k, v = O.seeded_qkv(1, 4, 256, 64, torch.float32)
    params = _config_like(4, 2, 3, 5, 0.1, torch.float32)
    want = _oracle_mta(q, k, v, params)
    mod = _mta_module(pkg, 4, 3, 5, 3, 3, *params, torch.float32)
    got = mod(q.cuda(), k.cuda(), v.cuda(), None, None)
    assert got.shape == (1, 256, 4, 64) and not got.is_contiguous()
    torch.testing.assert_close(got.cpu(), want, **tol(torch.float32))


@pytest.mark.parametrize("structure", ["infer", "dense", "probe"])
@pytest.mark.parametrize("post", ["identity", "random"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_mta_general(pkg, dtype, post, structure):
    print(f"mta general {dtype} post={post} structure={structure}", flush=True)
    q, k, v = O.seeded_qkv(2, 8, 200, 64, dtype)
    params = _config_like(8, 4, 6, 11, 0.05, dtype, post=post)
    want = _oracle_mta(q, k, v, params)
    mod = _mta_module(pkg, 8, 6, 11, 3, 3, *params, dtype, structure=structure)
    got = mod(q.cuda(), k.cuda(), v.cuda(), None, None).cpu()
    torch.testing.assert_close(got.float(), want.float(), **tol(dtype))


def test_mta_dense_head_weights(pkg):
    print("mta dense", flush=True)
    dtype = torch.float32
    q, k, v = O.seeded_qkv(1, 16, 96, 64, dtype)
    g = torch.Generator().manual_seed(5)
    params = [O.seeded_conv_weight(16, 3, 3, 0.1, dtype), torch.eye(16) + 0.1 * torch.randn(16, 16, generator=g),
              O.seeded_conv_weight(16, 3, 3, 0.1, dtype, seed=9), torch.eye(16) + 0.1 * torch.randn(16, 16, generator=g)]
    want = _oracle_mta(q, k, v, params)
    mod = _mta_module(pkg, 16, 3, 3, 3, 3, *params, dtype)
    got = mod(q.cuda(), k.cuda(), v.cuda(), None, None).cpu()
    torch.testing.assert_close(got, want, **tol(dtype))


def test_mta_identity_weights_is_sdpa(pkg):
    """The reference's own check (compare_mta_attention.py:21-27, 61-74): B2 H16 S128 D64 fp32, seed 123."""
    print("mta identity", flush=True)
    cfg = pkg.MTAConfig()
    mod = pkg.MTAAttentionTriton(16, cfg, 0.0, True).cuda().eval()
    mod.reset_mta_parameters()
    q, k, v = O.seeded_qkv(2, 16, 128, 64, torch.float32, seed=123)
    want = F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2)
    stages = []
    mod._stage_hook = stages.append
    got = mod(q.cuda(), k.cuda(), v.cuda(), None, None)     # parameters require grad: operator by operator
    assert stages == ["qk", "conv_pre", "mix_pre", "softmax", "conv_post", "mix_post", "pv", "end"]
    assert got.grad_fn is not None
    torch.testing.assert_close(got.detach().cpu(), want, rtol=1e-3, atol=1e-5)  # the reference script's own bar
    torch.testing.assert_close(got.detach().cpu(), want, **tol(torch.float32))
    with torch.no_grad():                                    # inference: fused route, dense weights assumed
        got = mod(q.cuda(), k.cuda(), v.cuda(), None, None).cpu()
    torch.testing.assert_close(got, want, **tol(torch.float32))
    assert mod.infer_weight_structure() == pkg.WeightStructure(True, 1, True, True, 1)
    with torch.no_grad():
        got = mod(q.cuda(), k.cuda(), v.cuda(), None, None).cpu()
    torch.testing.assert_close(got, want, **tol(torch.float32))


def test_mta_use_mask_path(pkg):
    print("mta use_mask", flush=True)
    dtype = torch.float32
    q, k, v = O.seeded_qkv(1, 4, 64, 64, dtype)
    params = _config_like(4, 2, 3, 5, 0.1, dtype, post="random")
    want = _oracle_mta(q, k, v, params)
    cfg = pkg.MTAConfig(query_kernel_size=3, key_kernel_size=5)
    mod = pkg.MTAAttentionTriton(4, cfg, 0.0, True, use_mask=True)
    with torch.no_grad():
        for dst, src in zip((mod.mta_conv_triton, mod.wpsm_triton, mod.mta_conv_after_sm_triton, mod.wposm_triton), params):
            dst.weight.copy_(src)
    mod = mod.cuda().eval()
    got = mod(q.cuda(), k.cuda(), v.cuda(), None, None).cpu()
    torch.testing.assert_close(got, want, **tol(dtype))


CA_CASES = [
    # B, H, S, D, R, Sk, causal, dtype
    (2, 8, 128, 64, 3, 3, True, torch.float32),     # compare_conv_attention2.py:106-125 shape, seed 42
    (1, 2, 300, 64, 6, 11, True, torch.float32),
    (1, 2, 257, 128, 6, 11, True, torch.bfloat16),
    (1, 3, 200, 128, 5, 7, False, torch.bfloat16),
    (1, 2, 130, 64, 1, 1, True, torch.float16),
    (1, 1, 64, 64, 2, 2, True, torch.float32),
    (1, 2, 500, 128, 11, 15, True, torch.float32),
    (1, 1, 1, 64, 3, 3, True, torch.float32),
    (1, 2, 1000, 128, 6, 11, True, torch.bfloat16),
    # 16-bit, kernel sizes with an all-MFMA instantiation
    (2, 2, 300, 64, 3, 3, True, torch.bfloat16),
    (1, 2, 515, 64, 5, 5, True, torch.float16),
    (1, 2, 260, 128, 7, 7, False, torch.bfloat16),
    (1, 2, 777, 128, 6, 11, True, torch.float16),
    (1, 1, 64, 128, 5, 7, True, torch.bfloat16),
    (1, 2, 5, 64, 6, 11, True, torch.bfloat16),
]


@pytest.mark.parametrize("case", CA_CASES)
def test_conv_attention_parity(pkg, case):
    b, h, s, d, r, sk, causal, dtype = case
    print(f"conv_attention case={case}", flush=True)
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=42)
    w = O.seeded_conv_weight(h, r, sk, 0.05, dtype)
    want = O.conv_attention_forward(q, k, v, w, causal, None)
    mod = pkg.TritonConvAttention(h, (r, sk), causal=causal)
    with torch.no_grad():
        mod.weight.copy_(w)
    mod = mod.to(dtype).cuda()
    got, qk = mod(q.cuda(), k.cuda(), v.cuda(), causal, d ** -0.5)
    assert qk is None and got.shape == q.shape and got.is_contiguous()
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dtype))


def test_conv_attention_identity_tap_is_sdpa(pkg):
    print("conv_attention identity", flush=True)
    q, k, v = O.seeded_qkv(2, 8, 128, 64, torch.float32, seed=42)
    w = O.identity_conv_kernel(8, 3, 3)
    for causal in (True, False):
        got = pkg.ops.conv_attn_fwd(q.cuda(), k.cuda(), v.cuda(), w.cuda(), causal, None).cpu()
        want = F.scaled_dot_product_attention(q, k, v, is_causal=causal)
        torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-5)


def test_conv_attention_row_slabs_long_sequence(pkg):
    """S=4096 bf16 6x11: compare three row slabs with the slab form of the oracle."""
    print("conv_attention slabs", flush=True)
    dtype = torch.bfloat16
    q, k, v = O.seeded_qkv(1, 2, 4096, 128, dtype)
    w = O.seeded_conv_weight(2, 6, 11, 0.05, dtype)
    got = pkg.ops.conv_attn_fwd(q.cuda(), k.cuda(), v.cuda(), w.cuda(), True, None).cpu()
    for r0, r1 in [(0, 128), (2040, 2170), (3968, 4096)]:
        want = O.conv_attention_rows(q, k, v, w, r0, r1, True, None)
        torch.testing.assert_close(got[:, :, r0:r1].float(), want.float(), **tol(dtype))


QKC_CASES = [
    # B, H, S, D, R, Sk, causal, dtype
    (1, 2, 256, 128, 6, 11, True, torch.bfloat16),
    (2, 2, 520, 64, 3, 3, True, torch.bfloat16),
    (1, 2, 248, 128, 6, 11, True, torch.float16),
    (1, 1, 776, 128, 5, 7, False, torch.bfloat16),
    (1, 2, 8, 64, 6, 11, True, torch.bfloat16),
    (1, 1, 1000, 128, 7, 7, True, torch.bfloat16),
    # long enough for the key range of a query block to be split into several work items
    (1, 1, 2048, 128, 6, 11, True, torch.bfloat16),
    (1, 2, 1800, 64, 3, 3, True, torch.float16),
    (1, 1, 1544, 128, 5, 5, False, torch.bfloat16),
    # 11x15, the kernel size of the reference's own benchmark script (benchmark_mta_attention.py:12-15): 112-row query blocks
    (1, 2, 520, 64, 11, 15, True, torch.bfloat16),
    (1, 1, 1160, 128, 11, 15, True, torch.float16),
    (1, 1, 264, 128, 11, 15, False, torch.bfloat16),
]


@pytest.mark.parametrize("fill", [True, False])
@pytest.mark.parametrize("case", QKC_CASES)
def test_qk_conv_parity(pkg, case, fill):
    """scale*conv(mask0(QK^T)) vs the oracle's first two stages (mta_attention_pytorch.py:63-67)."""
    b, h, s, d, r, sk, causal, dtype = case
    print(f"qk_conv case={case} fill={fill}", flush=True)
    q, k, _ = O.seeded_qkv(b, h, s, d, dtype, seed=7)
    w = O.seeded_conv_weight(h, r, sk, 0.05, dtype)
    scale = float(torch.rsqrt(torch.tensor(float(d))))
    s0 = torch.matmul(q, k.transpose(2, 3)) * torch.rsqrt(torch.tensor(d))
    want = O.depthwise_conv(torch.tril(s0) if causal else s0, w, causal)
    sentinel = 12345.0
    buf = torch.full((b, h, s, s), sentinel, dtype=dtype, device="cuda")
    got = pkg.ops.qk_conv(q.cuda(), k.cuda(), w.cuda(), causal, scale, fill_upper=fill, out=buf)
    assert got is buf and got.shape == (b, h, s, s)
    got = got.cpu()
    low = torch.tril(torch.ones(s, s, dtype=torch.bool)) if causal else torch.ones(s, s, dtype=torch.bool)
    # scores of magnitude ~sqrt(d)*|w| pass through two 16-bit roundings: 2 ulp + atol
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
    torch.testing.assert_close(got[..., low].float(), want[..., low].float(), rtol=2 * ulp, atol=2e-2)
    if causal and fill:
        up = ~low
        assert (got[..., up] == 0).all() and not torch.signbit(got[..., up]).any()
    if causal and not fill:     # above the diagonal is unspecified: left alone, or zero where a tile straddles it
        up = got[..., ~low].float()
        assert ((up == torch.tensor(sentinel).to(dtype).float()) | (up == 0)).all()
        if s >= 512:            # ... and tiles wholly above the diagonal are never touched
            assert (got[..., 0, s - 64:].float() == torch.tensor(sentinel).to(dtype).float()).all()


def _band_first(kind, b, s, seed=3):
    """int32 (B,S) first visible key per row: a sliding window, packed documents (per batch entry), or ragged."""
    rows = torch.arange(s)
    if kind == "window":
        return (rows - 99).clamp(min=0).to(torch.int32).expand(b, s).contiguous()
    g = torch.Generator().manual_seed(seed)
    if kind == "documents":   # a document starts where the random cut points fall; a row sees its own document
        out = torch.zeros(b, s, dtype=torch.int32)
        for i in range(b):
            cuts = torch.sort(torch.randint(1, s, (5,), generator=g)).values
            start = torch.zeros(s, dtype=torch.int64)
            for c in cuts.tolist():
                start[c:] = c
            out[i] = start.to(torch.int32)
        return out
    lo = (torch.rand(b, s, generator=g) * (rows + 1)[None, :]).floor().to(torch.int32)   # any value in 0 .. row
    return torch.minimum(lo, rows.to(torch.int32)[None, :]).contiguous()


BAND_CASES = [
    # B, H, S, D, R, Sk, dtype, kind
    (1, 2, 520, 64, 3, 3, torch.bfloat16, "window"), (2, 2, 776, 128, 6, 11, torch.bfloat16, "documents"),
    (1, 2, 264, 128, 7, 7, torch.float16, "ragged"), (2, 1, 2048, 128, 6, 11, torch.bfloat16, "window"),
    (1, 2, 520, 64, 11, 15, torch.float16, "documents"), (1, 1, 1160, 64, 5, 5, torch.bfloat16, "ragged"),
]


@pytest.mark.parametrize("case", BAND_CASES)
def test_qk_conv_band_parity(pkg, case):
    """The first stage under a band mask: the scores of the keys a row does not see are 0 on the way into the conv
    (mta_attention_pytorch.py:63-67 with a mask tensor), here from one int32 per (batch entry, row)."""
    b, h, s, d, r, sk, dtype, kind = case
    print(f"qk_conv band case={case}", flush=True)
    q, k, _ = O.seeded_qkv(b, h, s, d, dtype, seed=8)
    w = O.seeded_conv_weight(h, r, sk, 0.05, dtype)
    first = _band_first(kind, b, s)
    keys = torch.arange(s)
    visible = (keys[None, None, :] >= first[:, :, None]) & (keys[None, None, :] <= keys[None, :, None])   # (B,S,S)
    scale = float(torch.rsqrt(torch.tensor(float(d))))
    s0 = torch.matmul(q, k.transpose(2, 3)) * torch.rsqrt(torch.tensor(d))
    want = O.depthwise_conv(s0.masked_fill(~visible[:, None], 0), w, True)
    got = pkg.ops.qk_conv(q.cuda(), k.cuda(), w.cuda(), True, scale, fill_upper=True, first_visible=first.cuda()).cpu()
    low = torch.tril(torch.ones(s, s, dtype=torch.bool))
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
    # (defined where a row sees the key; key blocks that no row of a query block sees are not even visited)
    seen = visible[:, None].expand(b, h, s, s)
    torch.testing.assert_close(got[seen].float(), want[seen].float(), rtol=2 * ulp, atol=2e-2)
    assert (got[..., ~low] == 0).all()
    # no band at all is the plain kernel, bit for bit
    zero = torch.zeros(b, s, dtype=torch.int32, device="cuda")
    plain = pkg.ops.qk_conv(q.cuda(), k.cuda(), w.cuda(), True, scale, fill_upper=True)
    assert torch.equal(pkg.ops.qk_conv(q.cuda(), k.cuda(), w.cuda(), True, scale, fill_upper=True, first_visible=zero), plain)
    with pytest.raises(ValueError):
        pkg.ops.qk_conv(q.cuda(), k.cuda(), w.cuda(), False, scale, first_visible=zero)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("weights", ["both", "first", "second"])
@pytest.mark.parametrize("group,s", [(4, 520), (2, 2304), (8, 264), (1, 1000), (16, 136), (4, 4096), (4, 1608), (8, 2048),
                                     (16, 1160), (16, 2560)])
def test_headmix_softmax_band_parity(pkg, group, s, weights, dtype):
    """mix -> `scores + mask` -> softmax -> mix (mta_attention_triton.py:75-85) for a band mask given as the first
    visible key of every row; with one weight and 16-bit data the packed kernel's band instances run."""
    print(f"headmix_softmax band group={group} s={s} weights={weights} {dtype}", flush=True)
    if s >= 4096 and (dtype == torch.float32 or weights == "both"):
        pytest.skip("the long rows are there for the one-weight 16-bit kernels")
    n, c = (1, 8) if s >= 2048 else (2, 16)
    if c % group:
        c = group
    g = torch.Generator().manual_seed(13)
    x = (torch.randn(n, c, s, s, generator=g) * 2).to(dtype)
    w1 = O.block_diag_head_weight(c, group, 0.1, g, dtype) if weights != "second" else None
    w2 = O.block_diag_head_weight(c, group, 0.1, g, dtype) if weights != "first" else None
    first = _band_first("ragged" if s < 2048 else "window", n, s, seed=5)
    keys = torch.arange(s)
    hidden = keys[None, None, :] < first[:, :, None]                                     # (N,S,S)
    s1 = O.head_linear(x, w1, True, float("-inf")) if w1 is not None else x.masked_fill(
        torch.triu(torch.ones(s, s, dtype=torch.bool), 1), float("-inf"))
    s2 = s1.masked_fill(hidden[:, None], float("-inf"))
    p0 = torch.softmax(s2.float(), -1).to(dtype)
    want = O.head_linear(p0, w2, True, 0.0) if w2 is not None else p0
    cu = lambda t: None if t is None else t.cuda()
    w1, w2 = cu(w1), cu(w2)
    got = pkg.ops.headmix_softmax(x.cuda(), w1, w2, True, group_size=group, first_visible=first.cuda()).cpu()
    up = torch.triu(torch.ones(s, s, dtype=torch.bool), 1)
    assert (got[..., up] == 0).all()
    t = tol(dtype)
    torch.testing.assert_close(got.float(), want.float(), rtol=t["rtol"] * 2, atol=2e-3 if dtype != torch.float32 else 1e-6)
    # a band that hides nothing is the entry point without one
    zero = torch.zeros(n, s, dtype=torch.int32, device="cuda")
    a = pkg.ops.headmix_softmax(x.cuda(), w1, w2, True, group_size=group, first_visible=zero)
    torch.testing.assert_close(a.float().cpu(), pkg.ops.headmix_softmax(x.cuda(), w1, w2, True, group_size=group).float().cpu(),
                               rtol=t["rtol"] * 2, atol=2e-3 if dtype != torch.float32 else 1e-6)


@pytest.mark.parametrize("case", [(2, 2, 776, 64, torch.bfloat16, "documents"), (1, 3, 2048, 128, torch.float16, "window"),
                                  (2, 1, 520, 128, torch.bfloat16, "ragged")])
def test_causal_pv_band_skips_only_zeros(pkg, case):
    """P V under a band mask: P is 0 ahead of a row's first visible key, and the key blocks no row of a query block sees
    are not read -- the same sums as the product over the whole triangle, bit for bit; poisoning what is skipped
    (NaN in the blocks no row sees) changes nothing."""
    b, h, s, d, dtype, kind = case
    print(f"causal_pv band case={case}", flush=True)
    g = torch.Generator().manual_seed(17)
    first = _band_first(kind, b, s)
    keys = torch.arange(s)
    visible = (keys[None, None, :] >= first[:, :, None]) & (keys[None, None, :] <= keys[None, :, None])
    logits = (torch.randn(b, h, s, s, generator=g) * 2).masked_fill(~visible[:, None], float("-inf"))
    p = torch.softmax(logits, -1).to(dtype).cuda()
    v = torch.randn(b, h, s, d, generator=g).to(dtype).cuda()
    want = pkg.ops.causal_pv(p, v, True)
    got = pkg.ops.causal_pv(p, v, True, first_visible=first.cuda())
    assert torch.equal(got, want)
    # blocks of 64 keys wholly ahead of the first key any row of a block of 128 query rows sees: never read
    poisoned = p.clone()
    for bi in range(b):
        for q0 in range(0, s, 128):
            k_first = int(first[bi, q0:q0 + 128].min()) // 64 * 64
            poisoned[bi, :, q0:q0 + 128, :k_first] = float("nan")
    assert torch.equal(pkg.ops.causal_pv(poisoned, v, True, first_visible=first.cuda()), want)


def test_band_route_never_reads_what_it_skips(pkg):
    """The three kernels of the band route chained by hand, each writing into a NaN-filled buffer: what the scores kernel
    leaves unwritten (blocks no row sees, everything above the diagonal) must not reach the output."""
    print("band route poisoned buffers", flush=True)
    dtype = torch.bfloat16
    b, h, s, d = 2, 4, 1032, 64
    ops = pkg.ops
    q, k, v = (t.cuda() for t in O.seeded_qkv(b, h, s, d, dtype, seed=98))
    w = O.seeded_conv_weight(h, 6, 11, 0.05, dtype).cuda()
    g = torch.Generator().manual_seed(3)
    w1 = O.block_diag_head_weight(h, 2, 0.1, g, dtype).cuda()
    w2 = O.block_diag_head_weight(h, 2, 0.1, g, dtype).cuda()
    first = _band_first("window", b, s).cuda()
    scale = float(torch.rsqrt(torch.tensor(float(d))))

    def run(poison):
        fill = float("nan") if poison else 0.0
        s1 = ops.qk_conv(q, k, w, True, scale, fill_upper=False, first_visible=first,
                         out=torch.full((b, h, s, s), fill, dtype=dtype, device="cuda"))
        p1 = ops.headmix_softmax(s1, w1, w2, True, group_size=2, fill_upper=False, first_visible=first,
                                 out=torch.full((b, h, s, s), fill, dtype=dtype, device="cuda"))
        return ops.causal_pv(p1, v, True, first_visible=first)

    clean, poisoned = run(False), run(True)
    assert torch.isfinite(poisoned.float()).all()
    assert torch.equal(clean, poisoned)


@pytest.mark.parametrize("kind", ["window", "documents"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_mta_use_mask_band_masks_run_through_the_kernels(pkg, kind, dtype):
    """use_mask=True with a (B,1,S,S) mask of the form "row p sees the keys first[p] .. p" (sliding window, packed
    documents), bool and additive: the mask becomes one int32 per (batch entry, row) and the forward stays on the
    three-kernel route; against the oracle given the mask tensor (mta_attention_triton.py:63-64, 77-83, 96-127)."""
    print(f"mta use_mask band {kind} {dtype}", flush=True)
    b, h, s, d = 2, 4, 1032, 64
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=96)
    params = _config_like(h, 2, 6, 11, 0.05, dtype, post="identity")
    first = _band_first(kind, b, s)
    keys = torch.arange(s)
    visible = ((keys[None, None, :] >= first[:, :, None]) & (keys[None, None, :] <= keys[None, :, None]))[:, None]   # (B,1,S,S)
    additive = torch.where(visible, 0.0, float("-inf")).to(dtype)
    want = O.mta_forward(q, k, v, params[0].unsqueeze(1), params[1], params[2].unsqueeze(1), params[3],
                         mask=additive.expand(b, h, s, s).contiguous())
    assert torch.isfinite(want.float()).all()
    mod = _mta_module(pkg, h, 6, 11, 3, 3, *params, dtype, use_mask=True, structure="infer")
    for mask in (visible, additive):
        stages = []
        mod._stage_hook = stages.append
        got = mod(q.cuda(), k.cuda(), v.cuda(), mask.cuda(), None).cpu()
        assert stages == ["qk_conv", "mix_softmax_mix", "pv", "end"]
        torch.testing.assert_close(got.float(), want.float(), **tol(dtype))
    # a mask with a hole in a row is no band: the single-stage kernels with three mask passes between them, same values
    # as the oracle's
    holed = visible.clone()
    holed[0, 0, 700:, 650] = False
    want = O.mta_forward(q, k, v, params[0].unsqueeze(1), params[1], params[2].unsqueeze(1), params[3],
                         mask=torch.where(holed, 0.0, float("-inf")).to(dtype).expand(b, h, s, s).contiguous())
    stages = []
    mod._stage_hook = stages.append
    got = mod(q.cuda(), k.cuda(), v.cuda(), holed.cuda(), None).cpu()
    assert "qk_conv" not in stages and stages.count("mask") >= 2, stages   # (2: no post-softmax conv, so no pass behind it)
    torch.testing.assert_close(got.float(), want.float(), **tol(dtype))


TRI_CASES = [
    # B, H, S, D, R, Sk, group, dtype, band kind, weights
    (2, 8, 520, 64, 6, 11, 4, torch.bfloat16, None, "both"), (1, 4, 1160, 128, 3, 3, 2, torch.float16, None, "first"),
    (1, 8, 264, 128, 7, 7, 8, torch.bfloat16, None, "second"), (1, 8, 2304, 64, 6, 11, 4, torch.bfloat16, None, "both"),
    (2, 4, 776, 128, 6, 11, 4, torch.bfloat16, "documents", "first"), (1, 4, 2048, 64, 5, 5, 2, torch.float16, "window", "second"),
    (1, 8, 520, 64, 11, 15, 8, torch.bfloat16, "ragged", "first"), (1, 4, 4096, 128, 6, 11, 4, torch.bfloat16, None, "both"),
    # groups of 16 heads (the matrix-core softmax kernel's row lists): rows of all three kinds, two groups
    (1, 16, 2304, 64, 7, 7, 16, torch.float16, None, "first"), (2, 32, 1160, 64, 3, 3, 16, torch.bfloat16, None, "both"),
    # groups of 16 heads under band masks
    (1, 16, 1160, 64, 7, 7, 16, torch.bfloat16, "documents", "first"), (1, 32, 2304, 64, 3, 3, 16, torch.float16, "window", "both"),
    # a sequence shorter than one padded row; the longest rows the 8-head kernel takes; a band with groups of 8
    (1, 2, 8, 128, 3, 3, 2, torch.bfloat16, None, "both"), (1, 8, 2048, 128, 5, 7, 8, torch.float16, None, "both"),
    (1, 16, 72, 64, 3, 3, 16, torch.bfloat16, None, "second"), (2, 8, 1032, 64, 7, 7, 8, torch.bfloat16, "window", "second"),
    # the longest rows any of the kernels takes (pairs of heads, four passes per wavefront)
    (1, 2, 8192, 64, 3, 3, 2, torch.bfloat16, None, "both"),
]


@pytest.mark.parametrize("case", TRI_CASES)
def test_triangular_layout_stages_equal_the_plane_layout(pkg, case):
    """The three kernels of the causal forward over score tensors in the triangular layout (lower triangle only, rows
    padded to 64 keys, the heads of a group interleaved by rows): the same values, bit for bit, as over (B,H,S,S)
    tensors, stage by stage; padding and whatever lies ahead of a band is never read (NaN there changes nothing)."""
    b, h, s, d, r, sk, group, dtype, kind, weights = case
    print(f"triangular layout case={case}", flush=True)
    ops = pkg.ops
    q, k, v = (t.cuda() for t in O.seeded_qkv(b, h, s, d, dtype, seed=61))
    g = torch.Generator().manual_seed(62)
    w = (torch.randn(h, r, sk, generator=g) * 0.2).to(dtype).cuda()
    w1 = O.block_diag_head_weight(h, group, 0.1, g, dtype).cuda() if weights in ("both", "first") else None
    w2 = O.block_diag_head_weight(h, group, 0.1, g, dtype).cuda() if weights in ("both", "second") else None
    first = _band_first(kind, b, s).cuda() if kind else None
    assert ops.tri_route_supported(q, k, w, group, w1, w2, kind is not None)
    scale = d ** -0.5
    rows = torch.arange(s, device="cuda")
    visible = rows[None, :] <= rows[:, None]                                                   # (S,S)
    visible = visible[None].expand(b, s, s) if first is None else visible[None] & (rows[None, None, :] >= first[:, :, None])
    visible = visible[:, None].expand(b, h, s, s)

    s_plane = ops.qk_conv(q, k, w, True, scale, fill_upper=False, first_visible=first)
    s_tri = ops.qk_conv_tri(q, k, w, scale, group, first_visible=first)
    assert s_tri.numel() == b * h * ops.tri_row_offset(s)
    assert torch.equal(ops.tri_unpack(s_tri, b, h, s, group)[visible], s_plane[visible])

    p_plane = ops.headmix_softmax(s_plane, w1, w2, True, group_size=group, fill_upper=False, first_visible=first)
    p_tri = ops.headmix_softmax_tri(s_tri, w1, w2, b, h, s, group, first_visible=first)
    lower = (rows[None, :] <= rows[:, None])[None, None].expand(b, h, s, s)
    assert torch.equal(ops.tri_unpack(p_tri, b, h, s, group)[lower], p_plane[lower])
    # the same from an input whose padding, and whatever a band hides, is NaN
    poisoned = ops.tri_pack(s_plane.masked_fill(~visible, float("nan")), group)
    assert torch.equal(ops.headmix_softmax_tri(poisoned, w1, w2, b, h, s, group, first_visible=first)[ops.tri_pack(lower.to(dtype), group, 0.0) > 0],
                       p_tri[ops.tri_pack(lower.to(dtype), group, 0.0) > 0])

    if kind is None:   # with a key bias (key masks): a few keys hidden, a few finite values
        kb = torch.zeros(b, s)
        kb[:, 3::7] = float("-inf")
        kb[:, 5::11] = -1.5
        kb[:, 0] = 0
        kb = kb.cuda()
        biased = ops.headmix_softmax(s_plane, w1, w2, True, group_size=group, fill_upper=False, key_bias=kb)
        assert torch.equal(ops.tri_unpack(ops.headmix_softmax_tri(s_tri, w1, w2, b, h, s, group, key_bias=kb), b, h, s, group)[lower],
                           biased[lower])
    if group == 16:   # the same stage from the triangular layout into planes (what a post-softmax conv takes)
        mixed = ops.headmix_softmax_tri(s_tri, w1, w2, b, h, s, group, out_planes=True, first_visible=first)
        assert torch.equal(mixed[lower], p_plane[lower])

    o_plane = ops.causal_pv(p_plane, v, True, first_visible=first)
    assert torch.equal(ops.causal_pv_tri(p_tri, v, group, first_visible=first), o_plane)
    assert torch.equal(ops.causal_pv_tri(ops.tri_pack(p_plane.masked_fill(~lower, float("nan")), group), v, group,
                                         first_visible=first), o_plane)


def test_mta_score_layouts_agree_general_route(pkg):
    """Dense 16-head weights and a post-softmax conv: the first score tensor in the triangular layout (the default) or in
    planes, the same stages and the same output bit for bit."""
    print("mta score layouts, general route", flush=True)
    dtype = torch.float16
    b, h, s, d = 1, 16, 1160, 128
    q, k, v = (t.cuda() for t in O.seeded_qkv(b, h, s, d, dtype, seed=73))
    g = torch.Generator().manual_seed(74)
    dense = lambda: (torch.eye(h) + 0.05 * torch.randn(h, h, generator=g)).to(dtype)
    conv = lambda: (torch.randn(h, 7, 7, generator=g) * 0.05).to(dtype)
    mod = _mta_module(pkg, h, 7, 7, 7, 7, conv(), dense(), conv(), dense(), dtype, structure="dense")
    outs, stages = {}, {}
    for layout in ("auto", "planes"):
        mod.score_layout = layout
        seen = []
        mod._stage_hook = seen.append
        outs[layout] = mod(q, k, v, None, None)
        stages[layout] = seen
    assert stages["auto"] == stages["planes"] == ["qk_conv", "mix_softmax", "conv_mix_post", "pv", "end"]
    assert torch.equal(outs["auto"], outs["planes"])


@pytest.mark.parametrize("masked", [False, "band", "keys"])
def test_mta_score_layouts_agree(pkg, masked):
    """The module's inference route with the score tensors in the triangular layout (the default where the three kernels
    know it) and in planes: the same stages, the same output bit for bit - without a mask, under a sliding window and
    under a key-padding mask of a batch."""
    print(f"mta score layouts masked={masked}", flush=True)
    dtype = torch.bfloat16
    b, h, s, d = 2, 8, 1160, 128
    q, k, v = (t.cuda() for t in O.seeded_qkv(b, h, s, d, dtype, seed=71))
    params = _config_like(h, 4, 6, 11, 0.05, dtype)
    mod = _mta_module(pkg, h, 6, 11, 3, 3, *params, dtype, use_mask=bool(masked), structure="infer")
    mask = None
    rows = torch.arange(s)
    if masked == "band":
        mask = ((rows[None, :] <= rows[:, None]) & (rows[None, :] > rows[:, None] - 300))[None, None].cuda()
    elif masked == "keys":
        keep = rows[None, :] < torch.tensor([s, 700])[:, None]
        mask = (keep[:, None, None, :] & (rows[None, :] <= rows[:, None])[None, None]).cuda()
    outs, stages = {}, {}
    for layout in ("auto", "planes"):
        mod.score_layout = layout
        seen = []
        mod._stage_hook = seen.append
        outs[layout] = mod(q, k, v, mask, None)
        stages[layout] = seen
    assert stages["auto"] == stages["planes"] == ["qk_conv", "mix_softmax_mix", "pv", "end"]
    assert torch.equal(outs["auto"], outs["planes"])


@pytest.mark.parametrize("case", [(2, 8, 776, 64, 4, "documents", torch.bfloat16), (1, 16, 1160, 128, 16, "window", torch.float16),
                                  (1, 4, 520, 64, 2, "ragged", torch.bfloat16)])
def test_mta_use_mask_band_masks_with_a_post_softmax_conv(pkg, case):
    """Band masks with all four weights non-trivial (a 7x7 conv before and a 3x3 conv after the softmax, block-diagonal or
    dense head weights): the kernels run - scores under the band, softmax under the band, post-softmax conv, the hidden stretch of
    every row zeroed again (mta_attention_triton.py:82-83), head mixing, P V under the band - and the result is the
    oracle's given the mask tensor."""
    b, h, s, d, group, kind, dtype = case
    print(f"mta use_mask band + post conv case={case}", flush=True)
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=95)
    params = _config_like(h, group, 7, 7, 0.05, dtype, post="random")
    first = _band_first(kind, b, s)
    keys = torch.arange(s)
    visible = ((keys[None, None, :] >= first[:, :, None]) & (keys[None, None, :] <= keys[None, :, None]))[:, None]   # (B,1,S,S)
    want = O.mta_forward(q, k, v, params[0].unsqueeze(1), params[1], params[2].unsqueeze(1), params[3],
                         mask=torch.where(visible, 0.0, float("-inf")).to(dtype).expand(b, h, s, s).contiguous())
    mod = _mta_module(pkg, h, 7, 7, 3, 3, *params, dtype, use_mask=True, structure="infer")
    stages = []
    mod._stage_hook = stages.append
    got = mod(q.cuda(), k.cuda(), v.cuda(), visible.cuda(), None).cpu()
    assert stages[0] == "qk_conv" and "conv_post" in stages and stages[-2:] == ["pv", "end"], stages
    torch.testing.assert_close(got.float(), want.float(), **tol(dtype))


def test_mta_use_mask_key_padding_general_route(pkg):
    """Dense 16-head weights, a conv before and after the softmax, a key-padding mask of a batch: the four-kernel route
    (the matrix-core softmax kernel takes the key bias), against the oracle given the mask tensor."""
    print("mta use_mask key padding, general route", flush=True)
    dtype = torch.float16
    b, h, s, d = 2, 16, 776, 64
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=96)
    g = torch.Generator().manual_seed(97)
    dense = lambda: (torch.eye(h) + 0.05 * torch.randn(h, h, generator=g)).to(dtype)
    conv = lambda: (torch.randn(h, 7, 7, generator=g) * 0.05).to(dtype)
    params = [conv(), dense(), conv(), dense()]
    rows = torch.arange(s)
    keep = rows[None, :] < torch.tensor([s, 500])[:, None]
    visible = (keep[:, None, None, :] & (rows[None, :] <= rows[:, None])[None, None])
    want = O.mta_forward(q, k, v, params[0].unsqueeze(1), params[1], params[2].unsqueeze(1), params[3],
                         mask=torch.where(visible, 0.0, float("-inf")).to(dtype).expand(b, h, s, s).contiguous())
    mod = _mta_module(pkg, h, 7, 7, 7, 7, *params, dtype, use_mask=True, structure="dense")
    stages = []
    mod._stage_hook = stages.append
    got = mod(q.cuda(), k.cuda(), v.cuda(), visible.cuda(), None).cpu()
    assert stages == ["qk_conv", "mix_softmax", "conv_mix_post", "pv", "end"], stages
    torch.testing.assert_close(got.float(), want.float(), **tol(dtype))


def test_band_zero_clears_exactly_the_hidden_stretch(pkg):
    """mta_band_zero_fwd: x[n,c,p,q] = 0 for q < first[n,p], nothing else touched (not even NaN above the diagonal)."""
    print("band_zero", flush=True)
    for dtype, (n, c, s) in ((torch.bfloat16, (2, 3, 520)), (torch.float16, (1, 2, 72))):
        first = _band_first("ragged", n, s).cuda()
        first[:, 7] = 50                                     # beyond the diagonal: everything up to it is hidden
        x = torch.randn(n, c, s, s).to(dtype).cuda()
        x.masked_fill_(torch.triu(torch.ones(s, s, dtype=torch.bool, device="cuda"), 1), float("nan"))
        want = x.clone()
        keys = torch.arange(s, device="cuda")
        hidden = (keys[None, None, :] < first[:, :, None]) & (keys[None, None, :] <= keys[None, :, None])
        want.masked_fill_(hidden[:, None], 0)
        got = pkg.ops.band_zero_(x, first)
        assert got is x
        assert torch.equal(torch.nan_to_num(got, nan=123.0), torch.nan_to_num(want, nan=123.0))


def test_qk_conv_reports_unsupported(pkg):
    q = torch.zeros(1, 2, 64, 64, device="cuda")
    assert pkg.ops.qk_conv(q, q, torch.zeros(2, 3, 3, device="cuda"), True, 0.1) is None          # fp32
    qb = q.bfloat16()
    assert pkg.ops.qk_conv(qb, qb, torch.zeros(2, 9, 9, device="cuda").bfloat16(), True, 0.1) is None  # no 9x9 instance


PV_CASES = [(1, 2, 256, 128, True, torch.bfloat16), (2, 3, 520, 64, True, torch.float16), (1, 2, 1000, 128, True, torch.bfloat16),
            (1, 1, 264, 64, False, torch.bfloat16), (1, 2, 8, 128, True, torch.bfloat16)]


@pytest.mark.parametrize("case", PV_CASES)
def test_causal_pv_parity(pkg, case):
    b, h, s, d, causal, dtype = case
    print(f"causal_pv case={case}", flush=True)
    g = torch.Generator().manual_seed(3)
    logits = torch.randn(b, h, s, s, generator=g)
    if causal:
        logits.masked_fill_(torch.triu(torch.ones(s, s, dtype=torch.bool), 1), float("-inf"))
    p = torch.softmax(logits, -1).to(dtype)
    v = torch.randn(b, h, s, d, generator=g).to(dtype)
    want = torch.matmul(p, v)
    p_dev = p.cuda()
    if causal:  # what lies above the diagonal must never be read: poison it
        p_dev = p_dev.masked_fill(torch.triu(torch.ones(s, s, dtype=torch.bool, device="cuda"), 1), float("nan"))
    got = pkg.ops.causal_pv(p_dev, v.cuda(), causal)
    assert got is not None
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dtype))


PTX_CASES = [(1, 2, 256, 128, True, torch.bfloat16), (2, 3, 520, 64, True, torch.float16), (1, 2, 1000, 128, True, torch.bfloat16),
             (1, 1, 264, 64, False, torch.bfloat16), (1, 2, 8, 128, True, torch.float16), (1, 1, 2304, 128, True, torch.bfloat16),
             (1, 3, 136, 64, True, torch.bfloat16), (1, 1, 392, 128, False, torch.float16)]


@pytest.mark.parametrize("case", PTX_CASES)
def test_causal_ptx_parity(pkg, case):
    """out[k] = sum_{p >= k} P[p,k] X[p] (mta_causal_ptx_fwd: dV = P^T dO and dK = G^T Q of the training route) against
    the fp32 product of the same 16-bit values, with NaN above the diagonal of P: nothing there may be read."""
    b, h, s, d, causal, dtype = case
    print(f"causal_ptx case={case}", flush=True)
    g = torch.Generator().manual_seed(17)
    p = torch.randn(b, h, s, s, generator=g).to(dtype)
    x = torch.randn(b, h, s, d, generator=g).to(dtype)
    pm = torch.tril(p) if causal else p
    want = torch.matmul(pm.float().transpose(2, 3), x.float())
    p_dev = p.masked_fill(torch.triu(torch.ones(s, s, dtype=torch.bool), 1), float("nan")).cuda() if causal else p.cuda()
    got = pkg.ops.causal_ptx(p_dev, x.cuda(), causal)
    assert got is not None and got.dtype == dtype and got.shape == (b, h, s, d)
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    torch.testing.assert_close(got.cpu().float(), want, rtol=2 * ulp, atol=1e-3 * float(s) ** 0.5)


def test_mta_headline_config_small(pkg):
    """BASELINE config 4 at reduced S: bf16, 6x11 pre conv, identity post conv, groups of 4 -- the route
    qk_conv -> mix/softmax/mix -> causal P V, none of which writes or reads above the diagonal."""
    print("mta headline small", flush=True)
    dtype = torch.bfloat16
    q, k, v = O.seeded_qkv(2, 16, 512, 128, dtype)
    g = torch.Generator().manual_seed(125)
    params = [O.seeded_conv_weight(16, 6, 11, 0.05, dtype), torch.eye(16, dtype=dtype),
              O.identity_conv_kernel(16, 3, 3, dtype), O.block_diag_head_weight(16, 4, 0.1, g, dtype)]
    want = _oracle_mta(q, k, v, params)
    mod = _mta_module(pkg, 16, 6, 11, 3, 3, *params, dtype)
    stages = []
    mod._stage_hook = stages.append
    got = mod(q.cuda(), k.cuda(), v.cuda(), None, None).cpu()
    assert stages == ["qk_conv", "mix_softmax_mix", "pv", "end"]
    torch.testing.assert_close(got.float(), want.float(), **tol(dtype))


def test_mta_headline_route_long_sequence(pkg):
    """Same route at S=2048 (several work items per query block in the scores kernel, paired query blocks in P V)."""
    print("mta headline long", flush=True)
    dtype = torch.bfloat16
    q, k, v = O.seeded_qkv(1, 4, 2048, 128, dtype)
    g = torch.Generator().manual_seed(126)
    params = [O.seeded_conv_weight(4, 6, 11, 0.05, dtype), torch.eye(4, dtype=dtype),
              O.identity_conv_kernel(4, 3, 3, dtype), O.block_diag_head_weight(4, 4, 0.1, g, dtype)]
    want = _oracle_mta(q, k, v, params)
    mod = _mta_module(pkg, 4, 6, 11, 3, 3, *params, dtype)
    stages = []
    mod._stage_hook = stages.append
    got = mod(q.cuda(), k.cuda(), v.cuda(), None, None).cpu()
    assert stages == ["qk_conv", "mix_softmax_mix", "pv", "end"]
    torch.testing.assert_close(got.float(), want.float(), **tol(dtype))


def test_mta_headline_full_size(pkg):
    """BASELINE config 4 at its full size (B2 H16 S4096 D128 bf16, 6x11 pre conv, groups of 4).  The oracle is run on
    one mixing group of one batch element (the head mixing is block diagonal, so the slice is self-contained, and
    4 heads x 4096^2 scores is what the CPU finishes in seconds); every other (batch, head) is checked through the
    closed form of the first query row: one attended key, probability 1 for every head, so
    out[b,0,h,:] = bf16(sum_i wposm[h,i]) * v[b,h,0,:] (the output is laid out (B,S,H,D))."""
    print("mta headline full size", flush=True)
    dtype = torch.bfloat16
    b, h, s, d, grp = 2, 16, 4096, 128, 4
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=300)
    g = torch.Generator().manual_seed(127)
    params = [O.seeded_conv_weight(h, 6, 11, 0.05, dtype), O.block_diag_head_weight(h, grp, 0.1, g, dtype),
              O.identity_conv_kernel(h, 3, 3, dtype), O.block_diag_head_weight(h, grp, 0.1, g, dtype)]
    mod = _mta_module(pkg, h, 6, 11, 3, 3, *params, dtype)
    stages = []
    mod._stage_hook = stages.append
    got = mod(q.cuda(), k.cuda(), v.cuda(), None, None).cpu()
    assert stages == ["qk_conv", "mix_softmax_mix", "pv", "end"]
    assert torch.isfinite(got.float()).all()
    # closed form of query row 0, all batches and heads
    wsum = params[3].float().sum(dim=1).to(dtype).float()            # (H,) row sums of the post-softmax mix
    want0 = (wsum[None, :, None] * v[:, :, 0, :].float()).to(dtype)
    torch.testing.assert_close(got[:, 0, :, :].float(), want0.float(), **tol(dtype))
    # oracle on batch 1, heads 8..11
    bi, h0 = 1, 8
    sl = slice(h0, h0 + grp)
    sub = [params[0][sl], params[1][sl, sl], params[2][sl], params[3][sl, sl]]
    want = _oracle_mta(q[bi:bi + 1, sl], k[bi:bi + 1, sl], v[bi:bi + 1, sl], sub)
    torch.testing.assert_close(got[bi:bi + 1, :, sl].float(), want.float(), **tol(dtype))


def test_mta_forward_graph_capture_replay(pkg):
    """The forward route allocates through torch only and never synchronises, so it can be captured into a HIP graph.
    Every replay - with eager work and synchronisations between the replays - must reproduce the eager result bit
    for bit, also after the inputs have been overwritten in place."""
    print("mta graph capture", flush=True)
    dtype = torch.bfloat16
    h = 8
    g = torch.Generator().manual_seed(131)
    params = [O.seeded_conv_weight(h, 6, 11, 0.05, dtype), torch.eye(h, dtype=dtype),
              O.identity_conv_kernel(h, 3, 3, dtype), O.block_diag_head_weight(h, 4, 0.1, g, dtype)]
    mod = _mta_module(pkg, h, 6, 11, 3, 3, *params, dtype)
    q, k, v = [t.cuda() for t in O.seeded_qkv(1, h, 512, 128, dtype, seed=301)]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):          # warm up off the default stream, as torch asks before a capture
        for _ in range(2):
            mod(q, k, v, None, None)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = mod(q, k, v, None, None)
    torch.cuda.synchronize()
    for i in range(3):
        if i:                               # new inputs, written in place into the captured tensors
            q2, k2, v2 = O.seeded_qkv(1, h, 512, 128, dtype, seed=301 + i)
            q.copy_(q2.cuda()); k.copy_(k2.cuda()); v.copy_(v2.cuda())
        want = mod(q, k, v, None, None).clone()   # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {i} differs from the eager forward"


# ------------------------------------------------------------------------------------------------------
# weight structure is an opt-in: a rewritten parameter must never be served from stale assumptions
# ------------------------------------------------------------------------------------------------------
def test_mta_data_write_after_forward_is_seen(pkg):
    """Run with identity / block-diagonal weights, then overwrite the weights through ``.data`` (the reference's own
    idiom, mta_attention_triton.py:185-201) with dense ones and run again: the second result must follow the new
    weights, without any call that tells the module about the change."""
    print("mta .data write", flush=True)
    dtype = torch.bfloat16
    h = 8
    q, k, v = O.seeded_qkv(1, h, 256, 64, dtype, seed=77)
    g = torch.Generator().manual_seed(78)
    first = [O.seeded_conv_weight(h, 6, 11, 0.05, dtype), torch.eye(h, dtype=dtype),
             O.identity_conv_kernel(h, 3, 3, dtype), O.block_diag_head_weight(h, 4, 0.1, g, dtype)]
    second = [O.seeded_conv_weight(h, 6, 11, 0.05, dtype, seed=5),
              (torch.eye(h) + 0.1 * torch.randn(h, h, generator=g)).to(dtype),
              O.seeded_conv_weight(h, 3, 3, 0.05, dtype, seed=6),
              (torch.eye(h) + 0.1 * torch.randn(h, h, generator=g)).to(dtype)]
    for structure in ("dense", "probe"):
        mod = _mta_module(pkg, h, 6, 11, 3, 3, *first, dtype, structure=structure)
        got = mod(q.cuda(), k.cuda(), v.cuda(), None, None).cpu()
        torch.testing.assert_close(got.float(), _oracle_mta(q, k, v, first).float(), **tol(dtype))
        for dst, src in zip((mod.mta_conv_triton, mod.wpsm_triton, mod.mta_conv_after_sm_triton, mod.wposm_triton),
                            second):
            dst.weight.data.copy_(src)
        got = mod(q.cuda(), k.cuda(), v.cuda(), None, None).cpu()
        torch.testing.assert_close(got.float(), _oracle_mta(q, k, v, second).float(), **tol(dtype))
    # the explicit opt-in is dropped by the module's own ways of replacing parameters
    mod = _mta_module(pkg, h, 6, 11, 3, 3, *first, dtype, structure="infer")
    assert mod.weight_structure == "declared" and mod._declared.post_head_group == 4
    mod.load_state_dict({k_: v_.clone() for k_, v_ in mod.state_dict().items()})
    assert mod.weight_structure == "dense"


def test_weight_probes_on_device(pkg):
    print("weight probes", flush=True)
    ops = pkg.ops
    g = torch.Generator().manual_seed(0)
    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        w = torch.zeros(8, 8)
        for b in range(0, 8, 4):
            w[b:b + 4, b:b + 4] = torch.randn(4, 4, generator=g)
        assert ops.probe_head_weight(w.to(dtype).cuda()) == (False, 4)
        assert ops.probe_head_weight(torch.eye(8, dtype=dtype).cuda()) == (True, 1)
        assert ops.probe_head_weight((2 * torch.eye(8)).to(dtype).cuda()) == (False, 1)
        assert ops.probe_head_weight(torch.randn(6, 6, generator=g).to(dtype).cuda()) == (False, 6)
        w12 = torch.zeros(12, 12)
        w12[0:3, 0:3] = 1.0
        w12[3:6, 3:6] = 1.0
        w12[6:12, 6:12] = torch.randn(6, 6, generator=g)
        assert ops.probe_head_weight(w12.to(dtype).cuda()) == (False, 6)
        w12[11, 0] = 1e-3
        assert ops.probe_head_weight(w12.to(dtype).cuda()) == (False, 12)
        assert ops.probe_conv_kernel(O.identity_conv_kernel(5, 6, 11, dtype).cuda())
        assert ops.probe_conv_kernel(O.identity_conv_kernel(3, 1, 1, dtype).cuda())
        k = O.identity_conv_kernel(5, 6, 11, dtype)
        k[4, 0, 0] = 1e-3
        assert not ops.probe_conv_kernel(k.cuda())
        k = torch.zeros(2, 3, 4, dtype=dtype)
        k[:, -1, 2] = 1            # even key size: the tap is off by one, not a pass-through
        assert not ops.probe_conv_kernel(k.cuda())
        k = torch.zeros(2, 3, 3, dtype=dtype)
        k[:, 1, 1] = 1             # the module default (geometric centre) is not the pass-through tap
        assert not ops.probe_conv_kernel(k.cuda())
    assert ops.probe_head_weight(torch.eye(32).cuda() * float("nan")) == (False, 32)


# ------------------------------------------------------------------------------------------------------
# BASELINE configs at their full size, every head checked
# ------------------------------------------------------------------------------------------------------
def test_conv_attention_c5_full_size(pkg):
    """BASELINE config 5 at its real size: B1 H32 S8192 D128 bf16, 6x11, causal.  All 32 heads are compared with the
    slab form of the oracle on the first rows, on rows that cross the edge between two of the kernel's 248-row query
    blocks (248*17 = 4216), and on the last rows; query row 0 has the closed form o[0] = v[0]."""
    print("conv_attention C5 full size", flush=True)
    dtype = torch.bfloat16
    b, h, s, d = 1, 32, 8192, 128
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=500)
    w = O.seeded_conv_weight(h, 6, 11, 0.05, dtype)
    got = pkg.ops.conv_attn_fwd(q.cuda(), k.cuda(), v.cuda(), w.cuda(), True, None).cpu()
    assert torch.isfinite(got.float()).all()
    torch.testing.assert_close(got[:, :, 0].float(), v[:, :, 0].float(), rtol=0.0, atol=1e-6)
    for r0, r1 in [(0, 96), (4168, 4264), (8096, 8192)]:
        print(f"  slab {r0}:{r1}", flush=True)
        want = O.conv_attention_rows(q, k, v, w, r0, r1, True, None)
        torch.testing.assert_close(got[:, :, r0:r1].float(), want.float(), **tol(dtype))


def test_mta_headline_full_size_all_groups(pkg):
    """BASELINE config 4 at full size, every (batch, head): three row slabs (first rows; rows crossing the edge
    between two 248-row query blocks of the scores kernel, 248*8 = 1984; last rows) against the slab form of the
    oracle, which carries all 16 heads and both batch elements."""
    print("mta headline full size, all groups", flush=True)
    dtype = torch.bfloat16
    b, h, s, d, grp = 2, 16, 4096, 128, 4
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=300)
    g = torch.Generator().manual_seed(127)
    params = [O.seeded_conv_weight(h, 6, 11, 0.05, dtype), torch.eye(h, dtype=dtype),
              O.identity_conv_kernel(h, 3, 3, dtype), O.block_diag_head_weight(h, grp, 0.1, g, dtype)]
    mod = _mta_module(pkg, h, 6, 11, 3, 3, *params, dtype)
    stages = []
    mod._stage_hook = stages.append
    got = mod(q.cuda(), k.cuda(), v.cuda(), None, None).cpu()
    assert stages == ["qk_conv", "mix_softmax_mix", "pv", "end"]
    assert torch.isfinite(got.float()).all()
    for r0, r1 in [(0, 64), (1952, 2016), (4032, 4096)]:
        print(f"  slab {r0}:{r1}", flush=True)
        want = O.mta_forward_rows(q, k, v, params[0].unsqueeze(1), params[1], params[2].unsqueeze(1), params[3], r0, r1)
        torch.testing.assert_close(got[:, r0:r1].float(), want.float(), **tol(dtype))


def test_mta_headline_full_size_key_padding(pkg):
    """BASELINE config 4 at full size under a key-padding mask of the batch (lengths 4096 and 3000, a (B,1,S,S) boolean
    tensor; what bench.py times as its key-padding row).  Under the causal rule a row of a real token sees no padding
    key, so those rows must come out as without a mask, bit for bit - both batch entries, every head; the padding rows
    (whose own keys are hidden: they see the real tokens only) against the oracle on one mixing group."""
    print("mta headline full size, key padding", flush=True)
    dtype = torch.bfloat16
    b, h, s, d, grp = 2, 16, 4096, 128, 4
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=300)
    g = torch.Generator().manual_seed(127)
    params = [O.seeded_conv_weight(h, 6, 11, 0.05, dtype), torch.eye(h, dtype=dtype),
              O.identity_conv_kernel(h, 3, 3, dtype), O.block_diag_head_weight(h, grp, 0.1, g, dtype)]
    mod = _mta_module(pkg, h, 6, 11, 3, 3, *params, dtype, use_mask=True)
    plain = mod(q.cuda(), k.cuda(), v.cuda(), None, None)
    rows = torch.arange(s)
    lengths = torch.tensor([4096, 3000])
    mask = ((rows[None, :] < lengths[:, None])[:, None, None, :] & (rows[None, :] <= rows[:, None])[None, None]).cuda()
    stages = []
    mod._stage_hook = stages.append
    got = mod(q.cuda(), k.cuda(), v.cuda(), mask, None)
    assert stages == ["qk_conv", "mix_softmax_mix", "pv", "end"]
    assert torch.equal(got[0], plain[0]) and torch.equal(got[1, :3000], plain[1, :3000])
    assert torch.isfinite(got.float()).all()
    # the padding rows of batch entry 1, heads 4..7, against the oracle given the mask tensor (a slab of 64 rows)
    bi, sl, r0, r1 = 1, slice(4, 8), 3500, 3564
    sub = [params[0][sl], params[1][sl, sl], params[2][sl], params[3][sl, sl]]
    additive = torch.where(mask[bi:bi + 1].cpu(), 0.0, float("-inf")).to(dtype).expand(1, grp, s, s).contiguous()
    want = O.mta_forward(q[bi:bi + 1, sl], k[bi:bi + 1, sl], v[bi:bi + 1, sl], sub[0].unsqueeze(1), sub[1],
                         sub[2].unsqueeze(1), sub[3], mask=additive)
    torch.testing.assert_close(got[bi:bi + 1, r0:r1, sl].float().cpu(), want[:, r0:r1].float(), **tol(dtype))


# ------------------------------------------------------------------------------------------------------
# use_mask=True with real tensor masks, and the non-causal module
# ------------------------------------------------------------------------------------------------------
def _masks(s):
    g = torch.Generator().manual_seed(31)
    keep = torch.rand(1, s, generator=g) > 0.3
    keep[0, 0] = True                       # key 0 stays visible: no query row is fully blocked
    add = torch.zeros(1, 1, s, s)
    add.masked_fill_(torch.triu(torch.ones(s, s, dtype=torch.bool), 1), float("-inf"))
    add[0, 0, 40:, 9:23] = float("-inf")    # a block of keys hidden from the later rows
    boolean = torch.tril(torch.ones(s, s, dtype=torch.bool))[None, None].clone()
    boolean[0, 0, 5:, 2] = False
    return {"key_mask_bool": keep, "key_mask_additive": torch.where(keep, 0.0, float("-inf")),
            "additive_11SS": add, "bool_11SS": boolean}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", ["key_mask_bool", "key_mask_additive", "additive_11SS", "bool_11SS"])
def test_mta_use_mask_tensor_masks(pkg, name, dtype):
    """mta_attention_triton.py:63-64, 77-83, 96-127 with a mask tensor, vs the oracle given the same mask."""
    print(f"mta use_mask {name} {dtype}", flush=True)
    b, h, s, d = (1, 4, 136, 64)
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=91)
    params = _config_like(h, 2, 3, 5, 0.1, dtype, post="random")
    mask = _masks(s)[name]
    want = O.mta_forward(q, k, v, params[0].unsqueeze(1), params[1], params[2].unsqueeze(1), params[3], mask=mask)
    assert torch.isfinite(want.float()).all()
    for structure in ("dense", "infer"):
        mod = _mta_module(pkg, h, 3, 5, 3, 3, *params, dtype, use_mask=True, structure=structure)
        stages = []
        mod._stage_hook = stages.append
        got = mod(q.cuda(), k.cuda(), v.cuda(), mask.cuda(), None).cpu()
        torch.testing.assert_close(got.float(), want.float(), **tol(dtype))
        # a 2-D key mask runs through the kernels as a per-key bias in the softmax stage and zeroed K and V rows; a full
        # mask tensor with holes runs through the single-stage kernels with three mask passes between them
        assert "pv" in stages and (stages.count("mask") == 0) == name.startswith("key_mask"), stages
        assert name.startswith("key_mask") or stages.count("mask") == 3


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("group", [4, 16])
def test_mta_general_route_is_four_stages(pkg, group, dtype):
    """All four MTA weights non-trivial (what training produces): QK^T+conv, mix+softmax, conv+mix, P V -- four
    kernels, the score tensor written three times and read three times -- for mixing groups of 4 and for dense 16x16
    weights."""
    print(f"mta general route group={group} {dtype}", flush=True)
    h, s, d = 16, 520, 64
    q, k, v = O.seeded_qkv(1, h, s, d, dtype, seed=97)
    params = _config_like(h, group, 7, 7, 0.05, dtype, post="random")
    want = O.mta_forward(q, k, v, params[0].unsqueeze(1), params[1], params[2].unsqueeze(1), params[3])
    for structure in ("infer", "dense"):
        mod = _mta_module(pkg, h, 7, 7, 3, 3, *params, dtype, structure=structure)
        stages = []
        mod._stage_hook = stages.append
        got = mod(q.cuda(), k.cuda(), v.cuda(), None, None).cpu()
        # mixing groups of up to 4 heads, and dense groups of 16 at 16-bit dtypes (both halves on the matrix cores): the
        # post-softmax conv and the head mixing are one kernel
        assert stages == ["qk_conv", "mix_softmax", "conv_mix_post", "pv", "end"]
        torch.testing.assert_close(got.float(), want.float(), **tol(dtype))


@pytest.mark.parametrize("post", ["identity", "random"])
def test_mta_use_mask_key_mask_long_rows(pkg, post):
    """Key mask at a size where the 16-bit kernels run several passes per row (one-pass mix/softmax/mix and the
    stage-by-stage route), and use_mask=True without a mask tensor (the causal rule alone)."""
    print(f"mta use_mask key mask S=2304 post={post}", flush=True)
    dtype = torch.bfloat16
    b, h, s, d = 1, 4, 2304, 64
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=95)
    params = _config_like(h, 2, 6, 11, 0.05, dtype, post=post)
    g = torch.Generator().manual_seed(5)
    keep = torch.rand(1, s, generator=g) > 0.2
    keep[0, 0] = True
    for mask in (keep, None):
        want = O.mta_forward(q, k, v, params[0].unsqueeze(1), params[1], params[2].unsqueeze(1), params[3], mask=mask)
        mod = _mta_module(pkg, h, 6, 11, 3, 3, *params, dtype, use_mask=True, structure="infer")
        stages = []
        mod._stage_hook = stages.append
        got = mod(q.cuda(), k.cuda(), v.cuda(), None if mask is None else mask.cuda(), None).cpu()
        assert "qk_conv" in stages and "pv" in stages
        torch.testing.assert_close(got.float(), want.float(), **tol(dtype))


def test_mta_use_mask_key_mask_batched_additive_4d(pkg):
    """A (B,1,1,Sk)-style key mask cannot be expressed in the reference's 2-D form for B>1 (its repeat() stacks
    batches along the query axis, mta_attention_pytorch.py:130), so batches with different hidden keys arrive as a
    full (B,H,S,S) additive mask."""
    print("mta use_mask (B,H,S,S)", flush=True)
    dtype = torch.bfloat16
    b, h, s, d = 2, 4, 96, 64
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=92)
    params = _config_like(h, 4, 3, 3, 0.1, dtype, post="identity")
    g = torch.Generator().manual_seed(4)
    keep = torch.rand(b, s, generator=g) > 0.25
    keep[:, 0] = True
    causal = torch.tril(torch.ones(s, s, dtype=torch.bool))
    visible = (keep[:, None, None, :] & causal[None, None]).expand(b, h, s, s)
    mask = torch.where(visible, 0.0, float("-inf")).to(dtype).contiguous()
    want = O.mta_forward(q, k, v, params[0].unsqueeze(1), params[1], params[2].unsqueeze(1), params[3], mask=mask)
    mod = _mta_module(pkg, h, 3, 3, 3, 3, *params, dtype, use_mask=True)
    stages = []
    mod._stage_hook = stages.append
    got = mod(q.cuda(), k.cuda(), v.cuda(), mask.cuda(), None).cpu()
    torch.testing.assert_close(got.float(), want.float(), **tol(dtype))
    # "causal rule + hidden keys" per batch entry is recognised: the kernels run, with a key bias per batch entry
    assert "qk_conv" in stages and "pv" in stages


@pytest.mark.parametrize("post", ["identity", "random"])
def test_mta_use_mask_right_padded_batch(pkg, post):
    """Key padding for B > 1 (sequences of different lengths, padded on the right), given as a (B,1,S,S) boolean mask:
    recognised as "causal rule + hidden keys" and run through the kernels; the rows of real tokens against the oracle
    given the mask tensor (the padding rows see their own batch entry's kept keys only, like everybody else)."""
    print(f"mta use_mask right padding post={post}", flush=True)
    dtype = torch.bfloat16
    b, h, s, d = 3, 4, 520, 64
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=94)
    params = _config_like(h, 2, 6, 11, 0.05, dtype, post=post)
    lengths = torch.tensor([520, 333, 97])
    keep = torch.arange(s)[None, :] < lengths[:, None]                                  # (B,S)
    causal = torch.tril(torch.ones(s, s, dtype=torch.bool))
    visible = (keep[:, None, None, :] & causal[None, None])                            # (B,1,S,S)
    want = O.mta_forward(q, k, v, params[0].unsqueeze(1), params[1], params[2].unsqueeze(1), params[3],
                         mask=torch.where(visible, 0.0, float("-inf")).to(dtype).expand(b, h, s, s).contiguous())
    mod = _mta_module(pkg, h, 6, 11, 3, 3, *params, dtype, use_mask=True, structure="infer")
    stages = []
    mod._stage_hook = stages.append
    got = mod(q.cuda(), k.cuda(), v.cuda(), visible.cuda(), None).cpu()
    assert "qk_conv" in stages and "pv" in stages
    torch.testing.assert_close(got.float(), want.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("form", ["bool_BHSS", "additive_1HSS", "bool_B1SS"])
def test_mta_use_mask_arbitrary_planes(pkg, form, causal, dtype):
    """use_mask=True under masks of arbitrary content - random holes, a plane per head and / or per batch entry, boolean
    or 0 / -inf - for causal and non-causal modules: the single-stage kernels with the mask read as a byte per position in
    three passes (``mta_mask_fill_fwd``), against the oracle given the mask tensor.  Every row keeps a visible key (the
    diagonal)."""
    print(f"mta use_mask arbitrary planes {form} causal={causal} {dtype}", flush=True)
    b, h, s, d = 2, 4, 200, 64
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=99)
    params = _config_like(h, 2, 3, 5, 0.1, dtype, post="random")
    g = torch.Generator().manual_seed(100)
    shape = {"bool_BHSS": (b, h, s, s), "additive_1HSS": (1, h, s, s), "bool_B1SS": (b, 1, s, s)}[form]
    visible = torch.rand(shape, generator=g) > 0.3
    visible |= torch.eye(s, dtype=torch.bool)
    if causal:
        visible &= torch.tril(torch.ones(s, s, dtype=torch.bool))
    mask = torch.where(visible, 0.0, float("-inf")).to(dtype) if form.startswith("additive") else visible
    want = O.mta_forward(q, k, v, params[0].unsqueeze(1), params[1], params[2].unsqueeze(1), params[3],
                         mask=torch.where(visible, 0.0, float("-inf")).expand(b, h, s, s).contiguous())
    assert torch.isfinite(want.float()).all()
    mod = _mta_module(pkg, h, 3, 5, 3, 3, *params, dtype, causal=causal, use_mask=True, structure="dense")
    stages = []
    mod._stage_hook = stages.append
    got = mod(q.cuda(), k.cuda(), v.cuda(), mask.cuda(), None).cpu()
    assert stages == ["qk", "mask", "conv_pre", "mix_pre", "mask", "softmax", "conv_post", "mask", "mix_post", "pv", "end"], stages
    torch.testing.assert_close(got.float(), want.float(), **tol(dtype))
    # with the structure of the weights known, the block-diagonal head weights are applied by groups and identity stages
    # are skipped: an identity post-softmax conv and the mask pass behind it, an identity pre-softmax head weight
    for post, pre_eye, expect in (
            ("random", False, ["qk", "mask", "conv_pre", "mix_pre", "mask", "softmax", "conv_post", "mask", "mix_post", "pv", "end"]),
            ("identity", False, ["qk", "mask", "conv_pre", "mix_pre", "mask", "softmax", "mix_post", "pv", "end"]),
            ("identity", True, ["qk", "mask", "conv_pre", "mask", "softmax", "mix_post", "pv", "end"])):
        params2 = _config_like(h, 2, 3, 5, 0.1, dtype, post=post)
        if pre_eye:
            params2[1] = torch.eye(h, dtype=dtype)
        want2 = O.mta_forward(q, k, v, params2[0].unsqueeze(1), params2[1], params2[2].unsqueeze(1), params2[3],
                              mask=torch.where(visible, 0.0, float("-inf")).expand(b, h, s, s).contiguous())
        mod2 = _mta_module(pkg, h, 3, 5, 3, 3, *params2, dtype, causal=causal, use_mask=True, structure="infer")
        seen = []
        mod2._stage_hook = seen.append
        got2 = mod2(q.cuda(), k.cuda(), v.cuda(), mask.cuda(), None).cpu()
        assert seen == expect, seen
        torch.testing.assert_close(got2.float(), want2.float(), **tol(dtype))
    # an additive mask with finite values besides 0 and -inf: the same route, the mask itself added ahead of the softmax
    if form.startswith("additive"):
        g2 = torch.Generator().manual_seed(102)
        other = torch.where(visible, torch.randn(shape, generator=g2) * (torch.rand(shape, generator=g2) > 0.5), float("-inf"))
        other = other.to(dtype)
        want3 = O.mta_forward(q, k, v, params[0].unsqueeze(1), params[1], params[2].unsqueeze(1), params[3],
                              mask=other.expand(b, h, s, s).contiguous())
        del stages[:]
        got3 = mod(q.cuda(), k.cuda(), v.cuda(), other.cuda(), None).cpu()
        assert stages.count("mask") == 3, stages
        torch.testing.assert_close(got3.float(), want3.float(), **tol(dtype))


@pytest.mark.parametrize("case", [(2, 8, 520, 64, 4, 6, 11, "identity", torch.bfloat16), (2, 8, 264, 128, 4, 7, 7, "random", torch.float16),
                                  (2, 16, 1160, 64, 16, 3, 3, "identity", torch.bfloat16), (1, 16, 520, 128, 16, 7, 7, "random", torch.bfloat16),
                                  (2, 4, 2304, 64, 2, 6, 11, "identity", torch.float16)])
def test_mta_use_mask_left_padded_batch(pkg, case):
    """A left-padded batch (keys ahead of a sequence's start hidden; its padding rows therefore see nothing): a band mask
    whose empty rows have first[p] = p + 1.  It stays on the band route - the three kernels, or the general route with the
    empty rows of the probabilities cleared ahead of the post-softmax conv - and the padding rows' outputs are zeros, as
    the reference's masked_fill behind the softmax leaves them; against the oracle given the mask tensor."""
    b, h, s, d, group, r1, s1, post, dtype = case
    print(f"mta use_mask left padding {case}", flush=True)
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=104)
    params = _config_like(h, group, r1, s1, 0.05, dtype, post=post)
    pad = torch.tensor([0, s // 3][:b]) if b > 1 else torch.tensor([70])
    keep = torch.arange(s)[None, :] >= pad[:, None]
    visible = keep[:, None, None, :] & torch.tril(torch.ones(s, s, dtype=torch.bool))[None, None]     # keys only
    want = O.mta_forward(q, k, v, params[0].unsqueeze(1), params[1], params[2].unsqueeze(1), params[3],
                         mask=torch.where(visible, 0.0, float("-inf")).expand(b, h, s, s).contiguous())
    assert torch.isfinite(want.float()).all()
    mod = _mta_module(pkg, h, r1, s1, 3, 3, *params, dtype, use_mask=True, structure="infer")
    stages = []
    mod._stage_hook = stages.append
    got = mod(q.cuda(), k.cuda(), v.cuda(), visible.cuda(), None).cpu()
    assert "qk_conv" in stages and "mask" not in stages, stages
    if post == "identity":
        assert stages == ["qk_conv", "mix_softmax_mix", "pv", "end"], stages
    torch.testing.assert_close(got.float(), want.float(), **tol(dtype))
    last = b - 1
    assert not got[last, :int(pad[last])].any()


@pytest.mark.parametrize("post", ["identity", "random"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mta_use_mask_rows_that_see_nothing(pkg, dtype, post):
    """A left-padded batch whose mask hides the padding both as keys and as queries: the padding rows see no key at all.
    Their softmax is NaN; the reference zeroes it ahead of its post-softmax conv (mta_attention_triton.py:81), so their
    outputs are 0 and no other row is touched - the same here (one more mask pass behind the softmax), in inference and,
    with finite gradients that are zero for the padding, in training."""
    print(f"mta use_mask empty rows {dtype} post={post}", flush=True)
    b, h, s, d = 2, 4, 136, 64
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=103)
    params = _config_like(h, 2, 3, 5, 0.1, dtype, post=post)
    pad = torch.tensor([0, 37])
    keep = torch.arange(s)[None, :] >= pad[:, None]                                   # (B,S): left padding
    visible = (keep[:, None, :, None] & keep[:, None, None, :] & torch.tril(torch.ones(s, s, dtype=torch.bool))[None, None])
    want = O.mta_forward(q, k, v, params[0].unsqueeze(1), params[1], params[2].unsqueeze(1), params[3],
                         mask=torch.where(visible, 0.0, float("-inf")).expand(b, h, s, s).contiguous())
    assert torch.isfinite(want.float()).all() and not want[1, :37].any()
    for structure in ("dense", "infer"):
        mod = _mta_module(pkg, h, 3, 5, 3, 3, *params, dtype, use_mask=True, structure=structure)
        stages = []
        mod._stage_hook = stages.append
        got = mod(q.cuda(), k.cuda(), v.cuda(), visible.cuda(), None).cpu()
        assert stages.count("mask") == (4 if post == "random" or structure == "dense" else 3), stages
        torch.testing.assert_close(got.float(), want.float(), **tol(dtype))
        assert not got[1, :37].any()
    # training: the same forward, finite gradients, none for the padding
    mod = _mta_module(pkg, h, 3, 5, 3, 3, *params, dtype, use_mask=True, structure="dense").requires_grad_(True)
    qd, kd, vd = [t.clone().cuda().requires_grad_(True) for t in (q, k, v)]
    out = mod(qd, kd, vd, visible.cuda(), None)
    torch.testing.assert_close(out.detach().cpu().float(), want.float(), **tol(dtype))
    out.backward(torch.ones_like(out))
    for name, g_ in (("xq", qd.grad), ("xk", kd.grad), ("xv", vd.grad)):
        assert torch.isfinite(g_).all(), name
        assert not g_[1, :, :37].any(), f"the padding of {name} received a gradient"
    assert all(torch.isfinite(p_.grad).all() for p_ in mod.parameters())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_mask_fill_is_the_select(pkg, dtype):
    """ops.mask_fill against torch.where, bit for bit: 0 and -inf fills, in place and into another tensor, one mask plane
    for all or one per batch entry / head; with the causal rule nothing above the diagonal is touched."""
    print(f"mask_fill {dtype}", flush=True)
    n, c, p = 2, 3, 136
    g = torch.Generator().manual_seed(101)
    x = torch.randn(n, c, p, p, generator=g).to(dtype).cuda()
    low = torch.tril(torch.ones(p, p, dtype=torch.bool, device="cuda"))
    for shape in ((1, 1, p, p), (n, 1, p, p), (1, c, p, p), (n, c, p, p)):
        visible = (torch.rand(shape, generator=g) > 0.4).cuda()
        for neg_inf in (False, True):
            fill = float("-inf") if neg_inf else 0.0
            want = torch.where(visible, x, torch.tensor(fill, dtype=dtype, device="cuda"))
            got = pkg.ops.mask_fill(x, visible, neg_inf, False)
            assert torch.equal(got, want)
            poisoned = x.clone()
            poisoned[..., ~low] = float("nan")
            got = pkg.ops.mask_fill(poisoned, visible.view(torch.uint8), neg_inf, True, out=poisoned)
            assert got is poisoned and torch.equal(got[..., low], want[..., low]) and torch.isnan(got[..., ~low]).all()
    assert pkg.ops.mask_fill(x[..., :100].contiguous(), torch.ones(1, 1, p, 100, dtype=torch.bool, device="cuda"), False, False) is None
    # the additive pass: x + mask, rounded once, as torch adds two tensors of the dtype; -inf stays -inf
    for shape in ((1, 1, p, p), (n, c, p, p)):
        m = torch.randn(shape, generator=g).to(dtype).cuda()
        m[..., 3] = float("-inf")
        want = x + m
        assert torch.equal(pkg.ops.mask_add(x, m, False), want)
        poisoned = x.clone()
        poisoned[..., ~low] = float("nan")
        got = pkg.ops.mask_add(poisoned, m, True, out=poisoned)
        assert got is poisoned and torch.equal(got[..., low], want[..., low]) and torch.isnan(got[..., ~low]).all()


@pytest.mark.parametrize("kind", ["key_padding", "window"])
def test_mta_use_mask_probe_mode_follows_a_weight_rewrite(pkg, kind):
    """weight_structure = "probe" on the masked routes: the weights are looked at on every call, so a rewrite behind the
    module's back (block-diagonal post weights and an identity post conv replaced by dense ones through ``.data``) moves
    the next masked call from the three-kernel route to the general one, with the oracle's answer before and after."""
    print(f"mta use_mask probe mode {kind}", flush=True)
    dtype = torch.bfloat16
    b, h, s, d = 2, 8, 264, 64
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=97)
    g = torch.Generator().manual_seed(98)
    first = [O.seeded_conv_weight(h, 6, 11, 0.05, dtype), torch.eye(h, dtype=dtype),
             O.identity_conv_kernel(h, 3, 3, dtype), O.block_diag_head_weight(h, 4, 0.1, g, dtype)]
    second = [O.seeded_conv_weight(h, 6, 11, 0.05, dtype, seed=7),
              (torch.eye(h) + 0.1 * torch.randn(h, h, generator=g)).to(dtype),
              O.seeded_conv_weight(h, 3, 3, 0.05, dtype, seed=8),
              (torch.eye(h) + 0.1 * torch.randn(h, h, generator=g)).to(dtype)]
    pos = torch.arange(s)
    lower = pos[None, :] <= pos[:, None]
    if kind == "key_padding":
        keep = pos[None, :] < torch.tensor([264, 150])[:, None]
        visible = keep[:, None, None, :] & lower[None, None]
    else:
        visible = (lower & (pos[None, :] > pos[:, None] - 40))[None, None].expand(b, 1, s, s)
    full = visible.expand(b, h, s, s)
    mod = _mta_module(pkg, h, 6, 11, 3, 3, *first, dtype, use_mask=True, structure="probe")
    stages = []
    mod._stage_hook = stages.append
    got = mod(q.cuda(), k.cuda(), v.cuda(), visible.cuda(), None).cpu()
    want = O.mta_forward(q, k, v, first[0].unsqueeze(1), first[1], first[2].unsqueeze(1), first[3], mask=full)
    torch.testing.assert_close(got.float(), want.float(), **tol(dtype))
    assert stages == ["qk_conv", "mix_softmax_mix", "pv", "end"], stages
    for dst, src in zip((mod.mta_conv_triton, mod.wpsm_triton, mod.mta_conv_after_sm_triton, mod.wposm_triton), second):
        dst.weight.data.copy_(src)
    del stages[:]
    got = mod(q.cuda(), k.cuda(), v.cuda(), visible.cuda(), None).cpu()
    want = O.mta_forward(q, k, v, second[0].unsqueeze(1), second[1], second[2].unsqueeze(1), second[3], mask=full)
    torch.testing.assert_close(got.float(), want.float(), **tol(dtype))
    assert "conv_post" in stages or "conv_mix_post" in stages, stages


@pytest.mark.parametrize("post", ["identity", "random"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_mta_non_causal_key_padding(pkg, dtype, post):
    """MTAAttentionTriton(causal=False, use_mask=True) under key padding of a batch (a (B,1,S,S) boolean mask that hides
    the same keys from every row): recognised and run through the kernels' non-causal form with a key bias and zeroed K
    and V rows, no (B,H,S,S) mask tensor; against the oracle given the mask tensor.  A mask that is not of that form (a
    band) takes the composite."""
    print(f"mta causal=False key padding {dtype} post={post}", flush=True)
    b, h, s, d = 3, 4, 264, 64
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=96)
    params = _config_like(h, 2, 3, 5, 0.1, dtype, post=post)
    lengths = torch.tensor([264, 200, 31])
    keep = torch.arange(s)[None, :] < lengths[:, None]
    visible = keep[:, None, None, :].expand(b, 1, s, s).contiguous()
    want = O.mta_forward(q, k, v, params[0].unsqueeze(1), params[1], params[2].unsqueeze(1), params[3],
                         mask=visible.expand(b, h, s, s))
    for structure in ("dense", "infer"):
        mod = _mta_module(pkg, h, 3, 5, 3, 3, *params, dtype, causal=False, use_mask=True, structure=structure)
        seen = []
        classify = mod._structured_mask
        mod._structured_mask = lambda *a, f=classify: (seen.append(f(*a)) or seen[-1])
        got = mod(q.cuda(), k.cuda(), v.cuda(), visible.cuda(), None).cpu()
        assert seen and seen[-1][0] == "keys"
        torch.testing.assert_close(got.float(), want.float(), **tol(dtype))
    band = ((torch.arange(s)[:, None] - torch.arange(s)[None, :]).abs() <= 9)[None, None]
    assert classify(band.cuda(), b, s)[0] is None


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mta_non_causal_module(pkg, dtype):
    """MTAAttentionTriton(causal=False): no masking anywhere -- the oracle with an all-visible mask."""
    print(f"mta causal=False {dtype}", flush=True)
    b, h, s, d = 1, 4, 120, 64
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=93)
    params = _config_like(h, 2, 3, 5, 0.1, dtype, post="random")
    mask = torch.zeros(1, 1, s, s)
    want = O.mta_forward(q, k, v, params[0].unsqueeze(1), params[1], params[2].unsqueeze(1), params[3], mask=mask)
    for structure in ("dense", "infer"):
        mod = _mta_module(pkg, h, 3, 5, 3, 3, *params, dtype, causal=False, structure=structure)
        got = mod(q.cuda(), k.cuda(), v.cuda(), None, None).cpu()
        torch.testing.assert_close(got.float(), want.float(), **tol(dtype))
    # the same module with use_mask=True and a sliding-window mask (non-causal kernels, mask from the tensor only)
    band = ((torch.arange(s)[:, None] - torch.arange(s)[None, :]).abs() <= 9)[None, None]
    want = O.mta_forward(q, k, v, params[0].unsqueeze(1), params[1], params[2].unsqueeze(1), params[3], mask=band)
    mod = _mta_module(pkg, h, 3, 5, 3, 3, *params, dtype, causal=False, use_mask=True)
    got = mod(q.cuda(), k.cuda(), v.cuda(), band.cuda(), None).cpu()
    torch.testing.assert_close(got.float(), want.float(), **tol(dtype))


def test_conv_attention_general_kernel_bf16(pkg):
    """16-bit inputs with a kernel size that has no matrix-core conv instantiation (11x15) take the general kernel."""
    print("conv_attention general bf16", flush=True)
    for dtype in (torch.bfloat16, torch.float16):
        q, k, v = O.seeded_qkv(1, 2, 333, 128, dtype, seed=42)
        w = O.seeded_conv_weight(2, 11, 15, 0.05, dtype)
        want = O.conv_attention_forward(q, k, v, w, True, None)
        got = pkg.ops.conv_attn_fwd(q.cuda(), k.cuda(), v.cuda(), w.cuda(), True, None).cpu()
        torch.testing.assert_close(got.float(), want.float(), **tol(dtype))


def test_mta_unfused_16bit_route_never_reads_above_the_diagonal(pkg):
    """The stages of the 16-bit route that leave the upper triangle unwritten (scores kernel, mix+softmax with
    fill_upper=False) feed consumers that must not read it: run them into NaN-filled buffers and pass those on to
    the conv, the head mixing and P V."""
    print("mta poisoned upper triangle", flush=True)
    dtype = torch.bfloat16
    b, h, s, d = 1, 8, 264, 64
    ops = pkg.ops
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=95)
    w_pre, wpsm, w_post, wposm = _config_like(h, 4, 6, 11, 0.05, dtype, post="random")
    want = _oracle_mta(q, k, v, [w_pre, wpsm, w_post, wposm])
    nan = lambda: torch.full((b, h, s, s), float("nan"), dtype=dtype, device="cuda")
    scale = float(torch.rsqrt(torch.tensor(float(d))))
    s1 = ops.qk_conv(q.cuda(), k.cuda(), w_pre.cuda(), True, scale, fill_upper=False, out=nan())
    s1 = s1.masked_fill(torch.triu(torch.ones(s, s, dtype=torch.bool, device="cuda"), 1), float("nan"))
    p0 = ops.headmix_softmax(s1, wpsm.cuda(), None, True, group_size=4, out=nan(), fill_upper=False)
    up = torch.triu(torch.ones(s, s, dtype=torch.bool, device="cuda"), 1)
    assert (torch.isnan(p0[..., up]) | (p0[..., up] == 0)).all()
    p0 = p0.masked_fill(up, float("nan"))       # whatever the producer left there, the consumers must not read it
    p1 = ops.conv2d_causal(p0, w_post.cuda(), True)
    p2 = ops.headmix(p1, wposm.cuda(), True, 0.0, group_size=4)
    assert torch.isfinite(p2.float()).all() and (p2[..., up] == 0).all()
    p2 = p2.masked_fill(up, float("nan"))
    out = ops.causal_pv(p2, v.cuda(), True)
    torch.testing.assert_close(out.transpose(1, 2).cpu().float(), want.float(), **tol(dtype))


@pytest.mark.parametrize("h,group,dtype", [(8, 4, torch.bfloat16), (16, 16, torch.float16), (32, 32, torch.bfloat16)])
def test_mta_lower_triangle_route_never_reads_above_the_diagonal(pkg, h, group, dtype):
    """The inference route writes none of its intermediates above the diagonal (scores kernel and mix + softmax with
    fill_upper=False, mta_conv2d_tril_fwd, mta_headmix_tril_fwd).  Every stage here writes into a NaN-filled buffer
    and gets its input with the upper triangle set to NaN again: the result must be the oracle's."""
    print(f"mta lower-triangle route h={h} group={group} {dtype}", flush=True)
    b, s, d = 1, 264, 64
    ops = pkg.ops
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=96)
    w_pre, wpsm, w_post, wposm = _config_like(h, group, 6, 11, 0.05, dtype, post="random")
    want = _oracle_mta(q, k, v, [w_pre, wpsm, w_post, wposm])
    up = torch.triu(torch.ones(s, s, dtype=torch.bool, device="cuda"), 1)
    nan = lambda: torch.full((b, h, s, s), float("nan"), dtype=dtype, device="cuda")
    again = lambda t: t.masked_fill(up, float("nan"))
    scale = float(torch.rsqrt(torch.tensor(float(d))))
    x = again(ops.qk_conv(q.cuda(), k.cuda(), w_pre.cuda(), True, scale, fill_upper=False, out=nan()))
    if group <= 16:
        x = again(ops.headmix_softmax(x, wpsm.cuda(), None, True, group_size=group, out=nan(), fill_upper=False))
    else:
        x = again(ops.headmix(x, wpsm.cuda(), True, float("-inf"), group_size=group, out=nan(), fill_upper=False))
        x = again(ops.headmix_softmax(x, None, None, True, out=nan(), fill_upper=False))
    x = again(ops.conv2d_causal(x, w_post.cuda(), True, out=nan(), fill_upper=False))
    x = again(ops.headmix(x, wposm.cuda(), True, 0.0, group_size=group, out=nan(), fill_upper=False))
    assert torch.isfinite(x[..., ~up].float()).all()
    out = ops.causal_pv(x, v.cuda(), True)
    torch.testing.assert_close(out.transpose(1, 2).cpu().float(), want.float(), **tol(dtype))


@pytest.mark.parametrize("case", [(1, 2, 300, 64, 6, 11, True, torch.float32), (1, 2, 777, 128, 6, 11, True, torch.bfloat16),
                                  (2, 2, 260, 64, 3, 3, False, torch.float16), (1, 2, 333, 128, 11, 15, True, torch.bfloat16)])
def test_conv_attention_lse(pkg, case):
    """The row statistic of the fused kernel (the reference's M, conv_attention_triton.py:352-355, 402-404) against
    torch.logsumexp of the oracle's masked, scaled conv scores.  16-bit: the kernel rounds the conv output and the scaled
    logits to the I/O dtype (as the unfused pipeline stores them) and sums probabilities rounded to it, hence atol 2e-2."""
    b, h, s, d, r, sk, causal, dtype = case
    print(f"conv_attention lse case={case}", flush=True)
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=42)
    w = O.seeded_conv_weight(h, r, sk, 0.05, dtype)
    want = torch.logsumexp(O.conv_attention_scores(q.float(), k.float(), w.float(), causal, None), -1)
    o, lse = pkg.ops.conv_attn_fwd(q.cuda(), k.cuda(), v.cuda(), w.cuda(), causal, None, return_lse=True)
    assert lse.shape == (b, h, s) and lse.dtype == torch.float32
    t = dict(rtol=1e-4, atol=1e-4) if dtype == torch.float32 else dict(rtol=2.0 ** -7, atol=2e-2)
    torch.testing.assert_close(lse.cpu(), want, **t)
    o2 = pkg.ops.conv_attn_fwd(q.cuda(), k.cuda(), v.cuda(), w.cuda(), causal, None)
    assert torch.equal(o, o2)


def test_mta_general_route_published_shape_under_a_window_mask(pkg):
    """The published shape with all four weights non-trivial under a sliding-window mask tensor (what bench.py times as
    its general window row): the kernels run with the band (stage marks), and two size-independent checks against the
    unmasked forward of the same module - a window that hides nothing gives the same output (other kernels behind the
    softmax: to the usual tolerance), and under a 1024-key window the first 1024 rows, whose window hides nothing, are
    unchanged while later rows differ."""
    print("mta general route, published shape, window mask", flush=True)
    dtype = torch.float16
    b, h, s, d = 1, 16, 4096, 128
    q, k, v = (t.cuda() for t in O.seeded_qkv(b, h, s, d, dtype, seed=400))
    g = torch.Generator().manual_seed(321)
    params = [O.seeded_conv_weight(h, 7, 7, 0.05, dtype, seed=5), (torch.eye(h) + 0.1 * torch.randn(h, h, generator=g)).to(dtype),
              O.seeded_conv_weight(h, 7, 7, 0.05, dtype, seed=6), (torch.eye(h) + 0.1 * torch.randn(h, h, generator=g)).to(dtype)]
    mod = _mta_module(pkg, h, 7, 7, 7, 7, *params, dtype, use_mask=True, structure="dense")
    plain = mod(q, k, v, None, None)
    rows = torch.arange(s, device="cuda")
    causal = rows[None, :] <= rows[:, None]
    for width in (s, 1024):
        window = (causal & (rows[None, :] > rows[:, None] - width))[None, None]
        stages = []
        mod._stage_hook = stages.append
        got = mod(q, k, v, window, None)
        mod._stage_hook = None
        # (a window that hides nothing is "the causal rule and no hidden key": the route of key masks, with a zero bias)
        behind = ["conv_mix_post"] if width == s else ["conv_post", "mix_post"]
        assert stages == ["qk_conv", "mix_softmax", *behind, "pv", "end"], stages
        assert torch.isfinite(got.float()).all()
        same = slice(0, width)
        torch.testing.assert_close(got[:, same].float(), plain[:, same].float(), **tol(dtype))
        if width < s:
            assert (got[:, 2048:].float() - plain[:, 2048:].float()).abs().max() > 1e-2


@pytest.mark.parametrize("structure", ["infer", "dense"])
def test_mta_general_route_published_shape(pkg, structure):
    """The reference's published shape (benchmark_seq_len_results.jsonl: B1 H16 S4096 D128 fp16, 7x7 kernels before and
    after the softmax) with all four weights non-trivial and dense 16x16 head weights - what bench.py times as the
    general forward.  Three row slabs against the slab form of the oracle: the first rows; rows that cross an edge
    between two 120-row query blocks of the scores kernel (17*120 = 2040), the edge between two 128-row blocks of P V
    and the 2048-key boundary between two instances of the 16-head mix + softmax kernel; the last rows."""
    print(f"mta general route, published shape, structure={structure}", flush=True)
    dtype = torch.float16
    b, h, s, d = 1, 16, 4096, 128
    q, k, v = O.seeded_qkv(b, h, s, d, dtype, seed=400)
    g = torch.Generator().manual_seed(321)
    params = [O.seeded_conv_weight(h, 7, 7, 0.05, dtype, seed=5), (torch.eye(h) + 0.1 * torch.randn(h, h, generator=g)).to(dtype),
              O.seeded_conv_weight(h, 7, 7, 0.05, dtype, seed=6), (torch.eye(h) + 0.1 * torch.randn(h, h, generator=g)).to(dtype)]
    mod = _mta_module(pkg, h, 7, 7, 7, 7, *params, dtype, structure=structure)
    stages = []
    mod._stage_hook = stages.append
    got = mod(q.cuda(), k.cuda(), v.cuda(), None, None).cpu()
    assert stages[0] == "qk_conv" and "qk" not in stages and stages[-2:] == ["pv", "end"]
    assert "mix_softmax" in stages     # dense groups of 16 heads: mix + softmax on the matrix cores, one pass
    assert torch.isfinite(got.float()).all()
    for r0, r1 in [(0, 64), (2008, 2072), (4032, 4096)]:
        print(f"  slab {r0}:{r1}", flush=True)
        want = O.mta_forward_rows(q, k, v, params[0].unsqueeze(1), params[1], params[2].unsqueeze(1), params[3], r0, r1)
        torch.testing.assert_close(got[:, r0:r1].float(), want.float(), **tol(dtype))
