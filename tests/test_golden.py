"""Committed regression vectors (tests/golden/mta_golden.npz, written by make_golden.py).

CPU: the oracle still reproduces them (guards torch / oracle drift).
GPU: the HIP kernels, called through the C ABI, reproduce them without the oracle.
Tolerance: fp32 rtol 1e-4, atol 1e-5; fill patterns bit-exact.
"""
import os

import numpy as np
import pytest
import torch

from oracle import mta_oracle as O

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mta_golden.npz"))
TOL = dict(rtol=1e-4, atol=1e-5)


def t(name):
    return torch.from_numpy(GOLD[name])


def test_oracle_reproduces_golden():
    np.testing.assert_allclose(O.depthwise_conv(t("conv_x"), t("conv_w"), True).numpy(), GOLD["conv_y_causal"], **TOL)
    np.testing.assert_allclose(O.depthwise_conv(t("conv_x"), t("conv_w"), False).numpy(), GOLD["conv_y_full"], **TOL)
    np.testing.assert_allclose(O.head_linear(t("hm_x"), t("hm_w"), True, 0.0).numpy(), GOLD["hm_y_zero"], **TOL)
    got = O.head_linear(t("hm_x"), t("hm_w"), True, float("-inf")).numpy()
    assert np.array_equal(np.isneginf(got), np.isneginf(GOLD["hm_y_neginf"]))
    out = O.mta_forward(t("mta_q"), t("mta_k"), t("mta_v"), t("mta_w_pre").unsqueeze(1), t("mta_wpsm"),
                        t("mta_w_post").unsqueeze(1), t("mta_wposm"))
    np.testing.assert_allclose(out.numpy(), GOLD["mta_out"], **TOL)
    for causal, key in ((True, "ca_out_causal"), (False, "ca_out_full")):
        got = O.conv_attention_forward(t("ca_q"), t("ca_k"), t("ca_v"), t("ca_w"), causal, None)
        np.testing.assert_allclose(got.numpy(), GOLD[key], **TOL)


@pytest.mark.gpu
def test_kernels_reproduce_golden():
    import multitokenatention_triton_amd as mta
    ops = mta.ops
    dev = "cuda"
    for causal, key in ((True, "conv_y_causal"), (False, "conv_y_full")):
        got = ops.conv2d_causal(t("conv_x").to(dev), t("conv_w").to(dev), causal).cpu().numpy()
        np.testing.assert_allclose(got, GOLD[key], **TOL)
        if causal:
            up = np.triu(np.ones(got.shape[-2:], bool), 1)
            assert (got[..., up] == 0).all() and not np.signbit(got[..., up]).any()
    got = ops.headmix(t("hm_x").to(dev), t("hm_w").to(dev), True, 0.0).cpu().numpy()
    np.testing.assert_allclose(got, GOLD["hm_y_zero"], **TOL)
    got = ops.headmix(t("hm_x").to(dev), t("hm_w").to(dev), True, float("-inf")).cpu().numpy()
    assert np.array_equal(np.isneginf(got), np.isneginf(GOLD["hm_y_neginf"]))
    fin = np.isfinite(got)
    np.testing.assert_allclose(got[fin], GOLD["hm_y_neginf"][fin], **TOL)

    cfg = mta.MTAConfig(query_kernel_size=3, key_kernel_size=5)
    mod = mta.MTAAttentionTriton(4, cfg, 0.0, True)
    with torch.no_grad():
        mod.mta_conv_triton.weight.copy_(t("mta_w_pre"))
        mod.wpsm_triton.weight.copy_(t("mta_wpsm"))
        mod.mta_conv_after_sm_triton.weight.copy_(t("mta_w_post"))
        mod.wposm_triton.weight.copy_(t("mta_wposm"))
    mod = mod.to(dev).eval()
    # parameters require grad: the operator-by-operator route; then the fused inference route
    got = mod(t("mta_q").to(dev), t("mta_k").to(dev), t("mta_v").to(dev), None, None).detach().cpu().numpy()
    np.testing.assert_allclose(got, GOLD["mta_out"], **TOL)
    with torch.no_grad():
        got = mod(t("mta_q").to(dev), t("mta_k").to(dev), t("mta_v").to(dev), None, None).cpu().numpy()
    np.testing.assert_allclose(got, GOLD["mta_out"], **TOL)
    for causal, key in ((True, "ca_out_causal"), (False, "ca_out_full")):
        got = ops.conv_attn_fwd(t("ca_q").to(dev), t("ca_k").to(dev), t("ca_v").to(dev), t("ca_w").to(dev), causal, None)
        np.testing.assert_allclose(got.cpu().numpy(), GOLD[key], **TOL)
