"""CPU-only checks of the boundary: the C ABI library loads and exports what include/mta_hip.h declares,
argument validation returns the documented codes without touching a GPU, and the Python operator
surface mirrors the reference's names, parameters and error behaviour."""
import ctypes
import os
import re

import pytest
import torch

import multitokenatention_triton_amd as mta
from multitokenatention_triton_amd import _lib, ops

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mta_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mta_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = declared_functions()
    assert {"mta_conv2d_fwd", "mta_conv2d_scaled_fwd", "mta_headmix_fwd", "mta_headmix_softmax_fwd",
            "mta_conv_attn_fwd", "mta_qk_conv_fwd", "mta_causal_pv_fwd", "mta_strerror", "mta_abi_version",
            "mta_probe_head_weight", "mta_probe_conv_kernel"} <= set(names)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/mta_hip.h but not exported"
    assert sorted(_lib.SIGNATURES) == names, "ctypes signatures out of sync with the header"
    assert lib.mta_abi_version() == 10


def test_no_torch_symbols_in_the_library():
    out = os.popen(f"nm -D --undefined-only {_lib.LIB_PATH}").read()
    assert "at::" not in out and "c10" not in out and "torch" not in out


def test_error_strings():
    for code in range(0, -10, -1):
        s = _lib.strerror(code)
        assert s and "unknown" not in s
    assert "unknown" in _lib.strerror(-99)


def test_argument_validation_needs_no_gpu():
    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    p = ctypes.addressof(buf)
    # null pointers
    assert lib.mta_conv2d_fwd(None, p, p, 1, 1, 8, 8, 3, 3, 1, 0, 0, None) == -1
    assert lib.mta_headmix_fwd(p, None, p, 1, 2, 8, 8, 0, 1, 0.0, 0, 0, None) == -1
    assert lib.mta_conv_attn_fwd(p, p, p, p, None, 1, 1, 8, 64, 3, 3, 1, 0.1, 0, 0, None) == -1
    # dtype
    assert lib.mta_conv2d_fwd(p, p, p, 1, 1, 8, 8, 3, 3, 1, 7, 0, None) == -2
    # shape
    assert lib.mta_conv2d_fwd(p, p, p, 0, 1, 8, 8, 3, 3, 1, 0, 0, None) == -3
    # softmax gradient: null pointer, dtype, shape
    assert lib.mta_softmax_bwd(p, None, p, 1, 1, 8, 8, 1, 1, 0, None) == -1
    assert lib.mta_softmax_bwd(p, p, p, 1, 1, 8, 8, 1, 1, 9, None) == -2
    assert lib.mta_softmax_bwd(p, p, p, 1, 1, 8, 0, 1, 1, 0, None) == -3
    assert lib.mta_headmix_fwd(p, p, p, 1, 2, 0, 8, 0, 1, 0.0, 0, 0, None) == -3
    assert lib.mta_conv_attn_fwd(p, p, p, p, p, 1, 1, 0, 64, 3, 3, 1, 0.1, 0, 0, None) == -3
    # kernel size
    # (the conv operator takes up to 80 x 95 - the reference publishes rows for 77 x 77 -, the fused kernels up to 32 x 63)
    assert lib.mta_conv2d_fwd(p, p, p, 1, 1, 8, 8, 81, 3, 1, 0, 0, None) == -4
    assert lib.mta_conv2d_fwd(p, p, p, 1, 1, 8, 8, 3, 96, 1, 0, 0, None) == -4
    assert lib.mta_conv2d_bwd_input(p, p, p, 1, 1, 8, 8, 3, 96, 1, 0, 0, None) == -4
    assert lib.mta_conv_attn_fwd(p, p, p, p, p, 1, 1, 8, 64, 0, 3, 1, 0.1, 0, 0, None) == -4
    assert lib.mta_conv_attn_fwd(p, p, p, p, p, 1, 1, 8, 64, 33, 3, 1, 0.1, 0, 0, None) == -4
    assert lib.mta_qk_conv_fwd(p, p, p, p, 1, 1, 8, 64, 3, 64, 1, 0.1, 1, 1, 1, None) == -4
    assert b"80x95" in lib.mta_strerror(-4) and b"32x63" in lib.mta_strerror(-4)
    # group
    assert lib.mta_headmix_fwd(p, p, p, 1, 6, 8, 8, 4, 1, 0.0, 0, 0, None) == -5
    assert lib.mta_headmix_softmax_fwd(p, p, p, p, 1, 6, 8, 8, 4, 1, 1, 0, 0, None) == -5
    # combinations without a kernel are reported, not silently served by something else
    assert lib.mta_qk_conv_fwd(p, p, p, p, 1, 1, 8, 64, 3, 3, 1, 0.1, 1, 0, 0, None) == -9
    assert lib.mta_causal_pv_fwd(p, p, p, 1, 1, 8, 64, 1, 0, None) == -9
    assert lib.mta_causal_pv_fwd(p, p, p, 1, 1, 8, 48, 1, 1, None) == -7
    # alignment (fp32 pointer off by one byte)
    assert lib.mta_conv2d_fwd(p + 1, p, p, 1, 1, 8, 8, 3, 3, 1, 0, 0, None) == -6
    # head dim
    assert lib.mta_conv_attn_fwd(p, p, p, p, p, 1, 1, 8, 48, 3, 3, 1, 0.1, 0, 0, None) == -7


def test_triangular_layout_entry_points_validate_and_answer_on_the_host():
    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    p = ctypes.addressof(buf)
    # null pointers, group that does not divide the heads, dtypes without a kernel
    assert lib.mta_qk_conv_tri_fwd(p, p, p, None, None, 1, 4, 64, 64, 3, 3, 0.1, 4, 1, 1, None) == -1
    assert lib.mta_qk_conv_tri_fwd(p, p, p, None, p, 1, 6, 64, 64, 3, 3, 0.1, 4, 1, 1, None) == -5
    assert lib.mta_qk_conv_tri_fwd(p, p, p, None, p, 1, 4, 64, 64, 3, 3, 0.1, 4, 0, 0, None) == -9
    assert lib.mta_headmix_softmax_tri_fwd(None, p, p, None, None, p, 1, 4, 64, 4, 0, 1, 1, None) == -1
    assert lib.mta_headmix_softmax_tri_fwd(p, p, p, None, None, p, 1, 6, 64, 4, 0, 1, 1, None) == -5
    assert lib.mta_headmix_softmax_tri_fwd(p, p, p, None, None, p, 1, 4, 64, 4, 0, 0, 0, None) == -9      # fp32
    assert lib.mta_headmix_softmax_tri_fwd(p, None, None, None, None, p, 1, 4, 64, 4, 0, 1, 1, None) == -9  # no weight at all
    assert lib.mta_headmix_softmax_tri_fwd(p, p, p, p + 2, None, p, 1, 4, 64, 4, 0, 1, 1, None) == -6     # key bias off by 2 bytes
    assert lib.mta_causal_pv_tri_fwd(p, p, None, None, 1, 4, 64, 64, 4, 1, None) == -1
    assert lib.mta_causal_pv_tri_fwd(p, p, None, p, 1, 6, 64, 64, 4, 1, None) == -5
    assert lib.mta_causal_pv_tri_fwd(p, p, None, p, 1, 4, 64, 48, 4, 1, None) == -7
    assert lib.mta_band_zero_fwd(None, p, 1, 1, 8, 1, None) == -1 and lib.mta_band_zero_fwd(p, p, 1, 1, 8, 0, None) == -9
    assert lib.mta_band_zero_fwd(p, p, 1, 1, 12, 1, None) == -9 and lib.mta_band_zero_fwd(p, p, 0, 1, 8, 1, None) == -3
    # the mask pass: null pointers, a mask that is neither one plane nor one per batch entry / head, a width it does not take
    assert lib.mta_mask_fill_fwd(None, p, p, 1, 1, 8, 8, 1, 1, 0, 1, 1, None) == -1
    assert lib.mta_mask_fill_fwd(p, p, p, 2, 4, 8, 8, 3, 1, 0, 1, 1, None) == -3
    assert lib.mta_mask_fill_fwd(p, p, p, 2, 4, 8, 8, 1, 2, 0, 1, 1, None) == -3
    assert lib.mta_mask_fill_fwd(p, p, p, 1, 1, 8, 12, 1, 1, 0, 1, 1, None) == -9
    assert lib.mta_mask_add_fwd(None, p, p, 1, 1, 8, 8, 1, 1, 1, 1, None) == -1
    assert lib.mta_mask_add_fwd(p, p, p, 2, 4, 8, 8, 3, 1, 1, 1, None) == -3 and lib.mta_mask_add_fwd(p, p, p, 1, 1, 8, 12, 1, 1, 1, 1, None) == -9
    # which combinations the softmax stage has a kernel for: (C, S, group, out_planes, io, w, has_w1, has_w2, band, key_bias)
    q = lib.mta_headmix_softmax_tri_supported
    assert q(16, 4096, 4, 0, 1, 1, 1, 1, 0, 0) == 1 and q(16, 4104, 4, 0, 1, 1, 1, 1, 0, 0) == 0   # packed kernel: up to 4096 keys
    assert q(16, 8192, 2, 0, 2, 2, 1, 0, 0, 0) == 1 and q(16, 2048, 8, 0, 1, 1, 0, 1, 0, 0) == 1 and q(16, 2056, 8, 0, 1, 1, 0, 1, 0, 0) == 0
    assert q(16, 4096, 4, 0, 1, 1, 1, 0, 1, 0) == 1 and q(16, 4096, 4, 0, 1, 1, 1, 1, 1, 0) == 0   # band: one weight only
    assert q(16, 4096, 4, 0, 0, 0, 1, 1, 0, 0) == 0 and q(16, 4096, 4, 0, 1, 0, 1, 1, 0, 0) == 0   # fp32 data / fp32 weights
    assert q(16, 4096, 4, 1, 1, 1, 1, 1, 0, 0) == 0 and q(16, 4096, 16, 1, 1, 1, 1, 0, 0, 0) == 1   # planes out: groups of 16 only
    assert q(32, 4096, 16, 0, 2, 2, 1, 1, 0, 0) == 1 and q(32, 4096, 16, 0, 2, 2, 1, 1, 1, 0) == 1 and q(16, 4100, 16, 0, 1, 1, 1, 1, 0, 0) == 0
    assert q(16, 4096, 4, 0, 1, 1, 1, 1, 0, 1) == 1 and q(16, 4096, 4, 0, 1, 1, 1, 0, 1, 1) == 0 and q(16, 4096, 16, 0, 1, 1, 1, 1, 0, 1) == 1  # key bias
    # the layout's arithmetic: rows of 64*(p/64+1) elements, one after the other
    assert ops.tri_row_offset(0) == 0 and ops.tri_row_offset(1) == 64 and ops.tri_row_offset(64) == 4096
    assert ops.tri_row_offset(65) == 4096 + 128 and ops.tri_row_offset(4096) == sum(64 * (r // 64 + 1) for r in range(4096))


def test_check_maps_codes_to_exceptions():
    with pytest.raises(ValueError, match="kernel size"):
        _lib.check(-4, "x")
    with pytest.raises(RuntimeError):
        _lib.check(1, "x")
    _lib.check(0, "x")


def test_cpu_tensors_are_rejected_loudly():
    x = torch.zeros(1, 2, 8, 8)
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.conv2d_causal(x, torch.zeros(2, 3, 3), True)
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.headmix(x, torch.eye(2), True)
    with pytest.raises(RuntimeError, match="no CPU path"):
        mta.TritonConvAttention(2, 3)(torch.zeros(1, 2, 8, 64), torch.zeros(1, 2, 8, 64), torch.zeros(1, 2, 8, 64), True, 1.0)


def test_module_surface_matches_reference_names():
    cfg = mta.MTAConfig(query_kernel_size=6, key_kernel_size=11)
    mod = mta.MTAAttentionTriton(n_heads=8, mta=cfg, dropout=0.0, causal=True, use_mask=False)
    assert list(mod.state_dict()) == ["mta_conv_triton.weight", "wpsm_triton.weight",
                                      "mta_conv_after_sm_triton.weight", "wposm_triton.weight"]
    assert mod.mta_conv_triton.weight.shape == (8, 6, 11)
    assert mod.mta_conv_after_sm_triton.weight.shape == (8, 3, 3)
    assert mod.wpsm_triton.output_value == float("-inf") and mod.wposm_triton.output_value == 0.0
    # defaults of the operator modules (convolution_2d_trit.py:393-398, triton_linear_head.py:384)
    conv = mta.Conv2dTriton(4, (3, 5), causal=True)
    assert conv.weight[0, 1, 2] == 1 and conv.weight.sum() == 4
    assert mta.Conv2dTriton(4, 3).kernel_size == (3, 3)
    assert mta.TritonLinearHead(6).weight.shape == (6, 6)
    assert "head_dim=6" in repr(mta.TritonLinearHead(6))
    with pytest.raises(AssertionError, match="chunked"):
        mod(torch.zeros(1), torch.zeros(1), torch.zeros(1), None, chunk_start_ids=[0])


def test_reset_and_copy_parameters():
    cfg = mta.MTAConfig(query_kernel_size=3, key_kernel_size=5, init_method="identity")
    mod = mta.MTAAttentionTriton(4, cfg, 0.0, True)
    mod.reset_mta_parameters()
    w = mod.mta_conv_triton.weight
    assert w[0, 2, 2] == 1 and w.sum() == 4            # identity tap at [R-1, S//2]
    assert torch.equal(mod.wpsm_triton.weight, torch.eye(4)) and torch.equal(mod.wposm_triton.weight, torch.eye(4))

    class Src:  # the PyTorch module's parameter layout: conv kernels are (H,1,R,S)
        mta_kernel = torch.nn.Parameter(torch.randn(4, 1, 3, 5))
        mta_kernel_after_sm = torch.nn.Parameter(torch.randn(4, 1, 3, 3))
        wpsm = torch.nn.Linear(4, 4, bias=False)
        wposm = torch.nn.Linear(4, 4, bias=False)
    mod.copy_mta_parameters(Src)
    assert torch.equal(mod.mta_conv_triton.weight, Src.mta_kernel.squeeze(1))
    assert torch.equal(mod.wposm_triton.weight, Src.wposm.weight)
    # the other init modes (mta_attention_triton.py:150-183), each by its pattern
    for method in ("uniform", "normal", "diagonal", "const"):
        for r, sk in ((3, 5), (6, 11), (3, 3)):
            cfg = mta.MTAConfig(query_kernel_size=r, key_kernel_size=sk, init_method=method)
            m2 = mta.MTAAttentionTriton(4, cfg, 0.0, True)
            torch.manual_seed(7)
            m2.reset_mta_parameters()
            w, w2 = m2.mta_conv_triton.weight.detach(), m2.mta_conv_after_sm_triton.weight.detach()
            assert w.shape == (4, r, sk) and w2.shape == (4, 3, 3)
            assert torch.equal(m2.wpsm_triton.weight, torch.eye(4)) and torch.equal(m2.wposm_triton.weight, torch.eye(4))
            if method == "const":
                assert (w == 0.3).all() and (w2 == 0.3).all()
            elif method == "diagonal":
                # ones on the diagonal j - i = (S+1)//2 - R, which ends at the identity tap [R-1, S//2]; zero elsewhere
                i, j = torch.meshgrid(torch.arange(r), torch.arange(sk), indexing="ij")
                want = (j - i == (sk + 1) // 2 - r).float()
                assert want[r - 1, sk // 2] == 1 and want.sum() == min(r, sk // 2 + 1)
                assert torch.equal(w, want.expand(4, r, sk))
            elif method == "uniform":
                assert w.min() >= -1.0 and w.max() <= 1.0 and w.unique().numel() == w.numel()
                assert abs(float(w.mean())) < 0.5 and float(w.abs().max()) > 0.5
            else:   # "normal": std 0.3, truncated at three standard deviations
                assert w.abs().max() <= 0.9 and w.unique().numel() == w.numel() and 0.1 < float(w.std()) < 0.5
    cfg = mta.MTAConfig(query_kernel_size=3, key_kernel_size=5)
    cfg.init_method = "nope"
    with pytest.raises(ValueError):
        mta.MTAAttentionTriton(4, cfg, 0.0, True).reset_mta_parameters()


def test_weight_structure_is_an_opt_in():
    cfg = mta.MTAConfig()
    mod = mta.MTAAttentionTriton(4, cfg, 0.0, True)
    assert mod.weight_structure == "dense" and mod._current_structure() == mta.WeightStructure()
    st = mod.declare_weight_structure(pre_head_identity=True, post_conv_identity=True, post_head_group=2)
    assert mod.weight_structure == "declared" and mod._current_structure() is st
    assert st.post_head_group == 2 and st.pre_head_group is None and not st.post_head_identity
    with pytest.raises(ValueError, match="does not divide"):
        mod.declare_weight_structure(post_head_group=3)
    # every way the module itself replaces parameters drops the declaration
    mod.reset_mta_parameters()
    assert mod.weight_structure == "dense"
    mod.declare_weight_structure(post_head_group=2)
    mod.load_state_dict(mod.state_dict())
    assert mod.weight_structure == "dense"
    mod.declare_weight_structure(post_head_group=2)
    mod.copy_mta_parameters(object())
    assert mod.weight_structure == "dense"
    mod.weight_structure = "sometimes"
    with pytest.raises(ValueError, match="weight_structure"):
        mod._current_structure()
    with pytest.raises(RuntimeError, match="no CPU path"):      # the probes run on the device only
        mod.infer_weight_structure()


def test_forward_route_follows_grad_mode():
    """With grad enabled and parameters that require grad the module runs operator by operator (so that a graph is
    recorded); otherwise it takes the fused route.  Neither has a CPU path, so both stop at their first kernel - which is
    announced to the stage hook only if the library has it: the one-kernel scores stage for 16-bit data, the matrix
    product and the scaled conv for fp32 (mta_qk_conv_supported is a host-side question)."""
    lib = _lib.load()
    assert lib.mta_qk_conv_supported(4096, 128, 6, 11, 1, 1) == 1 and lib.mta_qk_conv_supported(4096, 128, 11, 15, 2, 2) == 1
    assert lib.mta_qk_conv_supported(4096, 128, 6, 11, 0, 0) == 0      # fp32
    assert lib.mta_qk_conv_supported(4096, 128, 6, 11, 1, 0) == 0      # weights of another dtype
    assert lib.mta_qk_conv_supported(4100, 128, 6, 11, 1, 1) == 0      # rows not whole 16-byte vectors
    assert lib.mta_qk_conv_supported(4096, 96, 6, 11, 1, 1) == 0 and lib.mta_qk_conv_supported(4096, 128, 9, 9, 1, 1) == 0
    for dtype, first in ((torch.float32, ["qk", "conv_pre"]), (torch.bfloat16, ["qk_conv"])):
        mod = mta.MTAAttentionTriton(4, mta.MTAConfig(), 0.0, True).to(dtype)
        x = torch.zeros(1, 4, 8, 64, dtype=dtype)
        seen = []
        mod._stage_hook = seen.append
        with pytest.raises(RuntimeError, match="no CPU path"):
            mod(x, x, x, None, None)                  # parameters require grad: operator by operator
        assert seen == first
        seen.clear()
        with torch.no_grad(), pytest.raises(RuntimeError, match="no CPU path"):
            mod(x, x, x, None, None)                  # fused route
        assert seen == first
        seen.clear()
        mod.requires_grad_(False)
        with pytest.raises(RuntimeError, match="no CPU path"):
            mod(x, x, x, None, None)
        assert seen == first
        seen.clear()
        with pytest.raises(RuntimeError, match="no CPU path"):
            mod(x.clone().requires_grad_(True), x, x, None, None)
        assert seen == first


def test_dropin_shims_resolve():
    import importlib
    import sys
    sys.path.insert(0, os.path.join(ROOT, "multitokenatention_triton_amd", "dropin"))
    try:
        m = importlib.import_module("mta_attention_triton")
        assert m.MTAAttentionTriton is mta.MTAAttentionTriton
        assert importlib.import_module("conv_attention_triton").TritonConvAttention is mta.TritonConvAttention
        assert importlib.import_module("convolution_2d_trit").Conv2dTriton is mta.Conv2dTriton
        assert importlib.import_module("triton_linear_head").TritonLinearHead is mta.TritonLinearHead
    finally:
        sys.path.pop(0)
