"""Pins the oracle (oracle/mta_oracle.py) without running the reference.

The torch-library restatement is checked against (a) brute-force nested loops in C,
(b) scipy's correlate2d, (c) closed forms: delta kernel == shift, identity tap ==
tril bit-exact, linearity, identity weights == causal SDPA, row 0 == V[0], and
(d) its own slab form.  Each check is chosen so that a flipped kernel, a wrong pad
side, a transposed head weight or a misplaced scale fails at least one of them.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F
from scipy.signal import correlate2d

from oracle import c_oracle
from oracle import mta_oracle as O


def _rand(shape, seed, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return std * torch.randn(*shape, generator=g)


@pytest.mark.parametrize("R,S", [(1, 1), (3, 3), (3, 5), (6, 11), (2, 7), (4, 4), (5, 6)])
@pytest.mark.parametrize("causal", [True, False])
def test_conv_vs_c_loops(R, S, causal):
    x = _rand((2, 3, 13, 13), 1)
    if causal:
        x = torch.tril(x)
    w = _rand((3, R, S), 2)
    got = O.depthwise_conv(x, w, causal).numpy()
    want = c_oracle.conv2d(x.numpy(), w.numpy(), causal)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)
    if causal:
        up = np.triu(np.ones((13, 13), bool), 1)
        assert (got[..., up] == 0).all() and not np.signbit(got[..., up]).any()


def test_conv_vs_scipy_correlate():
    x = _rand((1, 2, 9, 9), 3)
    w = _rand((2, 3, 5), 4)
    got = O.depthwise_conv(x, w, False).numpy()
    for c in range(2):
        padded = np.pad(x[0, c].numpy(), ((2, 0), (2, 2)))
        want = correlate2d(padded, w[c].numpy(), mode="valid")
        np.testing.assert_allclose(got[0, c], want, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("i,j", [(0, 0), (2, 4), (1, 2), (2, 2)])
def test_conv_delta_kernel_is_shift(i, j):
    R, S = 3, 5
    x = torch.tril(_rand((1, 1, 10, 10), 5))
    w = torch.zeros(1, R, S)
    w[0, i, j] = 1.0
    got = O.depthwise_conv(x, w, True)[0, 0]
    want = torch.zeros(10, 10)
    for p in range(10):
        for q in range(p + 1):
            h, k = p + i - (R - 1), q + j - (S - 1) // 2
            if 0 <= h < 10 and 0 <= k < 10 and k <= h:
                want[p, q] = x[0, 0, h, k]
    assert torch.equal(got, want)


def test_conv_identity_tap_is_tril_bit_exact():
    x = _rand((2, 4, 17, 17), 6)
    w = O.identity_conv_kernel(4, 6, 11)
    got = O.depthwise_conv(x, w, True)
    assert torch.equal(got, torch.tril(x) + 0.0)
    # the module-level conv (mask given, output not masked) agrees on the lower triangle
    mask = O.update_mask(None, 2, 4, x, 17)
    got2 = O.mta_convolution(x, mask, w.unsqueeze(1))
    assert torch.equal(torch.tril(got2), torch.tril(x))


def test_conv_linearity():
    x1, x2 = _rand((1, 2, 8, 8), 7), _rand((1, 2, 8, 8), 8)
    w1, w2 = _rand((2, 3, 3), 9), _rand((2, 3, 3), 10)
    f = lambda x, w: O.depthwise_conv(x, w, True)
    torch.testing.assert_close(f(x1 + x2, w1), f(x1, w1) + f(x2, w1), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(f(x1, w1 + w2), f(x1, w1) + f(x1, w2), rtol=1e-5, atol=1e-5)


def test_mta_convolution_equals_standalone_conv_on_lower_triangle():
    x = _rand((2, 3, 12, 12), 11)
    w = _rand((3, 4, 7), 12)
    mask = O.update_mask(None, 2, 3, x, 12)
    a = O.mta_convolution(x, mask, w.unsqueeze(1))
    b = O.depthwise_conv(torch.tril(x), w, True)
    torch.testing.assert_close(torch.tril(a), b, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("causal,fill", [(True, 0.0), (True, float("-inf")), (False, 0.0)])
def test_headmix_vs_c_loops(causal, fill):
    x = _rand((2, 6, 9, 9), 13)
    w = _rand((6, 6), 14)  # not symmetric: a transposed weight would fail
    got = O.head_linear(x, w, causal, fill).numpy()
    want = c_oracle.headmix(x.numpy(), w.numpy(), causal, fill)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)
    ein = torch.einsum("oi,bipq->bopq", w, x).numpy()
    low = np.tril(np.ones((9, 9), bool))
    np.testing.assert_allclose(got[..., low], ein[..., low], rtol=1e-5, atol=1e-5)


def test_headmix_identity_and_permutation_bit_exact():
    x = _rand((1, 4, 7, 7), 15)
    y = O.head_linear(x, torch.eye(4), True, 0.0)
    assert torch.equal(torch.tril(y), torch.tril(x))
    perm = torch.tensor([2, 0, 3, 1])
    wp = torch.zeros(4, 4)
    wp[torch.arange(4), perm] = 1.0  # y[o] = x[perm[o]]
    y = O.head_linear(x, wp, True, float("-inf"))
    assert torch.equal(torch.tril(y), torch.tril(x[:, perm]))
    assert torch.isneginf(y[..., torch.triu(torch.ones(7, 7, dtype=torch.bool), 1)]).all()


def _identity_params(h, r1, s1, r2, s2):
    return (O.identity_conv_kernel(h, r1, s1).unsqueeze(1), torch.eye(h),
            O.identity_conv_kernel(h, r2, s2).unsqueeze(1), torch.eye(h))


def test_mta_identity_weights_is_causal_sdpa():
    # the reference's own check: all-identity weights (compare_mta_attention.py:61-65)
    q, k, v = O.seeded_qkv(2, 4, 32, 16, torch.float32)
    out = O.mta_forward(q, k, v, *_identity_params(4, 3, 3, 3, 3))
    want = F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2)
    assert out.shape == (2, 32, 4, 16)
    torch.testing.assert_close(out, want, rtol=1e-5, atol=1e-6)


def test_mta_vs_c_restatement_config1_like():
    # B1 H4 S64 D16, 3x5 pre conv with identity tap, block-diag head weights, random post conv
    q, k, v = O.seeded_qkv(1, 4, 64, 16, torch.float32)
    g = torch.Generator().manual_seed(7)
    w_pre = O.seeded_conv_weight(4, 3, 5, 0.1, torch.float32)
    w_post = O.seeded_conv_weight(4, 2, 3, 0.1, torch.float32, seed=5)
    wpsm = O.block_diag_head_weight(4, 2, 0.1, g)
    wposm = O.block_diag_head_weight(4, 2, 0.1, g) + 0.05 * _rand((4, 4), 16)
    got = O.mta_forward(q, k, v, w_pre.unsqueeze(1), wpsm, w_post.unsqueeze(1), wposm).numpy()
    want = c_oracle.mta_forward(q.numpy(), k.numpy(), v.numpy(), w_pre.numpy(), wpsm.numpy(),
                                w_post.numpy(), wposm.numpy())
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-5)


def test_mta_row0_closed_form():
    # one unmasked key in row 0: softmax == 1 whatever the pre-softmax weights are
    q, k, v = O.seeded_qkv(1, 4, 16, 8, torch.float32)
    g = torch.Generator().manual_seed(3)
    w_pre = O.seeded_conv_weight(4, 6, 11, 0.05, torch.float32)
    wpsm = torch.eye(4) + 0.1 * torch.randn(4, 4, generator=g)
    wposm = torch.eye(4) + 0.1 * torch.randn(4, 4, generator=g)
    w_post = O.identity_conv_kernel(4, 3, 3)
    out = O.mta_forward(q, k, v, w_pre.unsqueeze(1), wpsm, w_post.unsqueeze(1), wposm)
    want = wposm.sum(1)[:, None] * v[0, :, 0, :]
    torch.testing.assert_close(out[0, 0], want, rtol=1e-5, atol=1e-6)


def test_mta_stages_compose_from_pinned_ops():
    q, k, v = O.seeded_qkv(1, 4, 24, 8, torch.float32)
    g = torch.Generator().manual_seed(11)
    w_pre = O.seeded_conv_weight(4, 3, 5, 0.1, torch.float32)
    w_post = O.seeded_conv_weight(4, 3, 3, 0.1, torch.float32, seed=9)
    wpsm = O.block_diag_head_weight(4, 2, 0.1, g)
    wposm = O.block_diag_head_weight(4, 2, 0.1, g)
    out, st = O.mta_forward(q, k, v, w_pre.unsqueeze(1), wpsm, w_post.unsqueeze(1), wposm,
                            return_stages=True)
    s0 = torch.matmul(q, k.transpose(2, 3)) * (8 ** -0.5)
    s1 = O.depthwise_conv(torch.tril(s0), w_pre, True)
    s2 = O.head_linear(s1, wpsm, True, float("-inf"))
    p0 = torch.softmax(s2, -1)
    p1 = O.depthwise_conv(p0, w_post, True)
    p2 = O.head_linear(p1, wposm, True, 0.0)
    want = torch.matmul(p2, v).transpose(1, 2)
    torch.testing.assert_close(out, want, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(torch.tril(st["s1"]), s1, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(st["p0"], p0, rtol=1e-5, atol=1e-6)


def test_mask_forms():
    x = torch.zeros(2, 3, 5, 8)
    causal = O.update_mask(None, 2, 3, x, 5)
    assert causal.shape == (2, 3, 5, 5)
    assert torch.equal(causal[0, 0] == 0, torch.tril(torch.ones(5, 5, dtype=torch.bool)))
    # a 2-D (B,Sk) key mask only keeps its shape for B=1: the reference's repeat()
    # (mta_attention_pytorch.py:130) stacks batches along the query axis otherwise.
    keep = torch.ones(1, 5, dtype=torch.bool)
    keep[0, 0] = False
    m = O.update_mask(keep, 1, 3, x[:1], 5)
    assert m.shape == (1, 3, 5, 5)
    assert torch.isneginf(m[0, :, :, 0]).all() and (m[0, :, 1:, 1] == 0).all()
    assert torch.isneginf(m[0, 0, 1, 2])
    one = torch.zeros(1, 1, 5, 5)
    assert O.update_mask(one, 2, 3, x, 5).shape == (2, 3, 5, 5)


@pytest.mark.parametrize("causal", [True, False])
def test_conv_attention_vs_c_restatement(causal):
    q, k, v = O.seeded_qkv(2, 3, 40, 16, torch.float32, seed=42)
    w = O.seeded_conv_weight(3, 4, 5, 0.1, torch.float32)
    got = O.conv_attention_forward(q, k, v, w, causal, 0.3).numpy()
    want = c_oracle.conv_attention(q.numpy(), k.numpy(), v.numpy(), w.numpy(), causal, 0.3)
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-5)


def test_conv_attention_identity_tap_is_sdpa():
    # compare_conv_attention2.py:106-136 shape and seed, identity kernel
    q, k, v = O.seeded_qkv(2, 8, 128, 64, torch.float32, seed=42)
    w = O.identity_conv_kernel(8, 3, 3)
    got = O.conv_attention_forward(q, k, v, w, True, None)
    want = F.scaled_dot_product_attention(q, k, v, is_causal=True)
    torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-5)
    got = O.conv_attention_forward(q, k, v, w, False, None)
    want = F.scaled_dot_product_attention(q, k, v, is_causal=False)
    torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-5)


def test_conv_attention_slab_form_equals_full_form():
    q, k, v = O.seeded_qkv(1, 2, 96, 16, torch.float32)
    w = O.seeded_conv_weight(2, 6, 11, 0.05, torch.float32)
    full = O.conv_attention_forward(q, k, v, w, True, None)
    for r0, r1 in [(0, 16), (3, 40), (80, 96)]:
        slab = O.conv_attention_rows(q, k, v, w, r0, r1, True, None)
        torch.testing.assert_close(slab, full[:, :, r0:r1], rtol=1e-5, atol=1e-6)


def test_conv_attention_is_composition_of_pinned_stages():
    q, k, v = O.seeded_qkv(1, 2, 32, 8, torch.float32)
    w = O.seeded_conv_weight(2, 3, 5, 0.1, torch.float32)
    s = torch.tril(torch.matmul(q, k.transpose(-1, -2)))
    c = O.depthwise_conv(s, w, True)
    c = c.masked_fill(torch.triu(torch.ones(32, 32, dtype=torch.bool), 1), float("-inf"))
    want = torch.matmul(torch.softmax(c * 0.25, -1), v)
    got = O.conv_attention_forward(q, k, v, w, True, 0.25)
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-6)


def test_mta_slab_form_equals_full_form():
    q, k, v = O.seeded_qkv(2, 4, 80, 16, torch.float32)
    g = torch.Generator().manual_seed(21)
    w_pre = O.seeded_conv_weight(4, 6, 11, 0.05, torch.float32).unsqueeze(1)
    w_post = O.seeded_conv_weight(4, 3, 3, 0.1, torch.float32, seed=9).unsqueeze(1)
    wpsm = O.block_diag_head_weight(4, 2, 0.1, g)
    wposm = O.block_diag_head_weight(4, 4, 0.1, g)
    full = O.mta_forward(q, k, v, w_pre, wpsm, w_post, wposm)
    for r0, r1 in [(0, 10), (3, 30), (7, 8), (64, 80)]:
        slab = O.mta_forward_rows(q, k, v, w_pre, wpsm, w_post, wposm, r0, r1)
        assert slab.shape == (2, r1 - r0, 4, 16)
        torch.testing.assert_close(slab, full[:, r0:r1], rtol=1e-5, atol=1e-6)


def _mask_cases(s):
    g = torch.Generator().manual_seed(31)
    keep = torch.rand(1, s, generator=g) > 0.3
    keep[0, 0] = True                       # key 0 stays visible: no query row is fully blocked
    add = torch.zeros(1, 1, s, s)
    add.masked_fill_(torch.triu(torch.ones(s, s, dtype=torch.bool), 1), float("-inf"))
    add[0, 0, 10:, 3:7] = float("-inf")     # a block of keys hidden from the later rows
    boolean = torch.tril(torch.ones(s, s, dtype=torch.bool))[None, None].clone()
    boolean[0, 0, 5:, 2] = False
    # non-causal shapes: a sliding window and a fully visible plane
    band = (torch.arange(s)[:, None] - torch.arange(s)[None, :]).abs() <= 6
    return {"key_mask_bool": keep, "additive_11SS": add, "bool_11SS": boolean,
            "band_bool": band[None, None], "all_visible": torch.zeros(1, 1, s, s)}


@pytest.mark.parametrize("name", ["key_mask_bool", "additive_11SS", "bool_11SS", "band_bool", "all_visible"])
def test_mta_tensor_masks_vs_c_restatement(name):
    """The explicit-mask branch of mta_forward (mta_attention_pytorch.py:58-83, 114-137) against the C loops
    given the additive mask that update_mask produces."""
    s = 24
    q, k, v = O.seeded_qkv(1, 4, s, 8, torch.float32, seed=55)
    g = torch.Generator().manual_seed(23)
    w_pre = O.seeded_conv_weight(4, 3, 5, 0.1, torch.float32)
    w_post = O.seeded_conv_weight(4, 2, 3, 0.1, torch.float32, seed=5)
    wpsm = O.block_diag_head_weight(4, 2, 0.1, g) + 0.05 * _rand((4, 4), 17)
    wposm = O.block_diag_head_weight(4, 2, 0.1, g)
    mask = _mask_cases(s)[name]
    got = O.mta_forward(q, k, v, w_pre.unsqueeze(1), wpsm, w_post.unsqueeze(1), wposm, mask=mask).numpy()
    add = O.update_mask(mask, 1, 4, q, s)
    assert add.shape == (1, 4, s, s) and not torch.isneginf(add).all(-1).any()
    want = c_oracle.mta_forward(q.numpy(), k.numpy(), v.numpy(), w_pre.numpy(), wpsm.numpy(), w_post.numpy(),
                                wposm.numpy(), mask=add.numpy())
    assert np.isfinite(got).all()
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-5)
    if name == "key_mask_bool":     # hidden keys and the causal rule both took effect
        hidden = (~mask[0]).nonzero().flatten()
        assert torch.isneginf(add[0, :, :, hidden]).all() and torch.isneginf(add[0, 0, 3, 4])


def test_conv_attention_scores_and_lse():
    q, k, v = O.seeded_qkv(1, 2, 40, 8, torch.float32, seed=3)
    w = O.seeded_conv_weight(2, 3, 5, 0.1, torch.float32)
    for causal in (True, False):
        sc = O.conv_attention_scores(q, k, w, causal, 0.3)
        lse = torch.logsumexp(sc, -1)
        p = torch.exp(sc - lse[..., None])
        torch.testing.assert_close(p.sum(-1), torch.ones(1, 2, 40), rtol=1e-5, atol=1e-6)
        torch.testing.assert_close(torch.matmul(p, v), O.conv_attention_forward(q, k, v, w, causal, 0.3),
                                   rtol=1e-5, atol=1e-6)
        if causal:   # row 0 sees one key: lse is that logit, scale * w[R-1, S//2] * (q0 . k0)
            want = 0.3 * w[:, -1, 2] * (q[0, :, 0] * k[0, :, 0]).sum(-1)
            torch.testing.assert_close(lse[0, :, 0], want, rtol=1e-5, atol=1e-6)


# ---------------------------------------------------------------------------------------
# backward of the two operators
# ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("rs", [(3, 3), (2, 5), (4, 4)])
def test_conv_grads_pinned(causal, rs):
    r, s = rs
    x, w, dy = _rand((2, 3, 9, 9), 41), _rand((3, r, s), 42), _rand((2, 3, 9, 9), 43)
    dx, dw = O.depthwise_conv_grads(x, w, causal, dy)
    # the reference's own backward kernels, as nested loops
    cdx, cdw = c_oracle.conv2d_bwd(x.numpy(), w.numpy(), dy.numpy(), causal)
    np.testing.assert_allclose(dx.numpy(), cdx, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(dw.numpy(), cdw, rtol=1e-5, atol=1e-5)
    # adjoint identities of an operator that is linear in x and in w
    y = O.depthwise_conv(x, w, causal)
    torch.testing.assert_close((y * dy).sum(), (x * dx).sum(), rtol=1e-4, atol=1e-4)
    torch.testing.assert_close((y * dy).sum(), (w * dw).sum(), rtol=1e-4, atol=1e-4)
    if causal:
        assert (dx.triu(1) == 0).all()
    # finite differences
    xd = x[:1, :, :6, :6].double().requires_grad_(True)
    wd = w.double().requires_grad_(True)
    assert torch.autograd.gradcheck(lambda a, b: O.depthwise_conv(a, b, causal), (xd, wd), eps=1e-6, atol=1e-6)


@pytest.mark.parametrize("causal,fill", [(True, 0.0), (True, float("-inf")), (False, 0.0)])
def test_headmix_grads_pinned(causal, fill):
    x, w, dy = _rand((2, 5, 7, 7), 51), _rand((5, 5), 52), _rand((2, 5, 7, 7), 53)
    dx, dw = O.head_linear_grads(x, w, causal, fill, dy)
    cdx, cdw = c_oracle.headmix_bwd(x.numpy(), w.numpy(), dy.numpy(), causal)
    np.testing.assert_allclose(dx.numpy(), cdx, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(dw.numpy(), cdw, rtol=1e-5, atol=1e-5)
    if causal:
        assert (dx.triu(1) == 0).all()
    if fill == 0.0:
        y = O.head_linear(x, w, causal, fill)
        live = torch.tril(torch.ones(7, 7)) if causal else torch.ones(7, 7)
        torch.testing.assert_close((y * dy * live).sum(), (w * dw).sum(), rtol=1e-4, atol=1e-4)
        xd, wd = x[:1].double().requires_grad_(True), w.double().requires_grad_(True)
        assert torch.autograd.gradcheck(lambda a, b: O.head_linear(a, b, causal, 0.0), (xd, wd), eps=1e-6, atol=1e-6)
