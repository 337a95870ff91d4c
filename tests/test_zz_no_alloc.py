"""kh_group_norm_static_bf16: the GroupNorm entry point that allocates nothing.

It keeps its partial statistics in an array the library holds on the GPU instead of a caller workspace.  The check is
bit equality with kh_group_norm_bf16 (same kernels) on two calls in a row, the second on a smaller input so that
partial sums left over from the first call would show if they were read, plus the fp32 oracle within the bf16
tolerance.  Both entry points are called through the C ABI with raw pointers.
"""
import pytest
import torch

from helpers import assert_close_rel, bf16_round

pytestmark = pytest.mark.gpu

BF = torch.bfloat16
REL_BF16 = 2e-2


def _ptr(t):
    return None if t is None else t.data_ptr()


def _call_both(lib, x, gamma, beta, add_nc, G, eps, act, channels_last):
    """(static-scratch result, caller-workspace result) for one input."""
    N, C, H, W = x.shape
    stream = torch.cuda.current_stream().cuda_stream
    nbytes = lib.kh_group_norm_workspace_bytes(N, C, H * W, G, channels_last)
    assert 0 < nbytes <= 256 * 1024
    ws = torch.empty(nbytes // 4, dtype=torch.float32, device=x.device)
    y_ws = torch.empty_like(x)
    rc = lib.kh_group_norm_bf16(_ptr(x), _ptr(y_ws), _ptr(gamma), _ptr(beta), _ptr(add_nc), _ptr(ws), N, C, H * W, G,
                                eps, act, channels_last, stream)
    assert rc == 0, lib.kh_error_string(rc)
    y_st = torch.empty_like(x)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    rc = lib.kh_group_norm_static_bf16(_ptr(x), _ptr(y_st), _ptr(gamma), _ptr(beta), _ptr(add_nc), N, C, H * W, G,
                                       eps, act, channels_last, stream)
    assert rc == 0, lib.kh_error_string(rc)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    return y_st, y_ws


@pytest.mark.parametrize("channels_last", [1, 0])
def test_static_group_norm_matches_workspace_entry_point(channels_last):
    from katz_amd import _lib
    from oracle import ops as O

    lib = _lib.load()
    d = torch.device("cuda:0")
    g = torch.Generator().manual_seed(7)
    # first a large input (2 x 640 x 64 x 64: many partial sums), then a smaller one with fewer splits
    for shape, G, act, with_add in (((2, 640, 64, 64), 32, 1, True), ((1, 320, 16, 16), 32, 0, False)):
        print("static group norm", shape, "nhwc" if channels_last else "nchw", flush=True)
        N, C, H, W = shape
        x = bf16_round(torch.randn(*shape, generator=g) * 2 + 0.5)
        gamma = bf16_round(1 + 0.1 * torch.randn(C, generator=g))
        beta = bf16_round(0.1 * torch.randn(C, generator=g))
        add = bf16_round(torch.randn(N, C, generator=g)) if with_add else None
        xd = x.to(d, BF)
        if channels_last:
            xd = xd.contiguous(memory_format=torch.channels_last)
        add_d = None if add is None else add.to(d, BF)
        y_st, y_ws = _call_both(lib, xd, gamma.to(d, BF), beta.to(d, BF), add_d, G, 1e-5, act, channels_last)
        assert torch.equal(y_st, y_ws)
        xin = x if add is None else x + add[:, :, None, None]
        ref = O.group_norm(xin, G, gamma, beta, 1e-5, "silu" if act else "none")
        assert_close_rel(y_st, ref, REL_BF16, "kh_group_norm_static_bf16")


def test_static_group_norm_rejects_what_does_not_fit():
    from katz_amd import _lib

    lib = _lib.load()
    # 600 samples x 512 groups need more than 256 KiB of partial sums: refused before any launch
    N, C, HW, G = 600, 4096, 64, 512
    assert lib.kh_group_norm_workspace_bytes(N, C, HW, G, 1) > 256 * 1024
    assert lib.kh_group_norm_static_bf16(16, 16, None, None, None, N, C, HW, G, 1e-5, 0, 1, None) == -4
    assert lib.kh_group_norm_static_bf16(None, 16, None, None, None, 2, 64, 64, 8, 1e-5, 0, 1, None) == -1
