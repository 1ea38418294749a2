"""The entry point that allocates nothing, mta_conv2d_bwd_weight_noalloc, called through the C ABI and compared with
mta_conv2d_bwd_weight (the entry point it is a variant of) on two calls in a row, the second with a smaller input.

Same kernels and -- when both use the same number of partial kernels -- the same order of additions: bit-exact.
With a large conv kernel the static array holds fewer partial kernels than the workspace of the other entry point, the
order differs and the bar is the fp32 one (rtol 1e-4, atol 1e-5 times the largest magnitude).
"""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _call_pair(lib, ops, x, dy, r, s, causal):
    n, c, h, w = x.shape
    want = ops.conv2d_bwd_weight(x, dy, (r, s), causal)
    got = torch.full((c, r, s), float("nan"), dtype=torch.float32, device=x.device)
    code = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}[x.dtype]
    rc = lib.mta_conv2d_bwd_weight_noalloc(x.data_ptr(), dy.data_ptr(), got.data_ptr(), n, c, h, w, r, s, int(causal), code,
                                           torch.cuda.current_stream().cuda_stream)
    assert rc == 0, rc
    return got, want


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_noalloc_matches_workspace_entry_point(dtype):
    from multitokenatention_triton_amd import _lib, ops
    lib = _lib.load()
    g = torch.Generator().manual_seed(11)
    shapes = [((2, 16, 512, 512), 6, 11), ((1, 4, 96, 96), 6, 11)]      # the second call is smaller than the first
    for rep in range(2):
        for shape, r, s in shapes:
            print(f"noalloc {shape} {r}x{s} {dtype} rep={rep}", flush=True)
            x = torch.randn(*shape, generator=g).to(dtype).cuda()
            dy = torch.randn(*shape, generator=g).to(dtype).cuda()
            got, want = _call_pair(lib, ops, x, dy, r, s, True)
            assert torch.equal(got, want)
    # a large kernel: fewer partial kernels fit the static array, so the order of additions differs
    x = torch.randn(1, 64, 128, 128, generator=g).to(dtype).cuda()
    dy = torch.randn(1, 64, 128, 128, generator=g).to(dtype).cuda()
    got, want = _call_pair(lib, ops, x, dy, 32, 63, False)
    torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-5 * float(want.abs().max()))
    got, want = _call_pair(lib, ops, x[:, :8, :40, :40].contiguous(), dy[:, :8, :40, :40].contiguous(), 3, 3, True)
    assert torch.equal(got, want)


def test_noalloc_rejects_what_does_not_fit():
    from multitokenatention_triton_amd import _lib
    lib = _lib.load()
    x = torch.zeros(1, 256, 8, 8, device="cuda")
    dw = torch.zeros(256, 32, 63, device="cuda")
    # 256 channels x 32 x 63 taps = 2 MiB of sums: more than the 1 MiB the library holds
    rc = lib.mta_conv2d_bwd_weight_noalloc(x.data_ptr(), x.data_ptr(), dw.data_ptr(), 1, 256, 8, 8, 32, 63, 1, 0, None)
    assert rc == -10 and "workspace" in _lib.strerror(rc)
