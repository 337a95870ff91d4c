"""The `fast_kernel` drop-in: torch.ops.fast_kernel.* with the reference's names and argument lists
(diffusers-hf/src/fast_kernel/fast_kernel/csrc/bind.cu:12-15; call sites models/normalization.py:90-91,
models/activations.py:145)."""
import pytest
import torch

from helpers import assert_close_rel, bf16_round

BF = torch.bfloat16


def test_install_registers_the_two_ops_and_the_module_name():
    import katz_amd.fast_kernel_shim as shim

    shim.install()
    shim.install()                       # idempotent
    import fast_kernel                   # what normalization.py:23 / activations.py:21 do

    assert fast_kernel is shim
    gn = torch.ops.fast_kernel.group_norm_fp16.default._schema
    assert [a.name for a in gn.arguments] == ["x", "y", "eps", "num_groups", "activation", "weight", "bias", "affine",
                                              "channels_last"]
    assert len(gn.returns) == 0
    gm = torch.ops.fast_kernel.fast_gelu_mul_fp16.default._schema
    assert [a.name for a in gm.arguments] == ["x", "m"] and len(gm.returns) == 1


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_group_norm_fp16_reference_call(dtype):
    """The exact call of normalization.py:90-91: NHWC x, caller-allocated y, "silu", last flag False."""
    import katz_amd.fast_kernel_shim as shim
    from oracle import ops as O

    shim.install()
    print("fast_kernel.group_norm_fp16", dtype, flush=True)
    g = torch.Generator().manual_seed(3)
    x = bf16_round(torch.randn(2, 320, 32, 32, generator=g) * 1.5 + 0.3)
    if dtype == torch.float16:
        x = x.half().float()
    w, b = bf16_round(1 + 0.1 * torch.randn(320, generator=g)), bf16_round(0.1 * torch.randn(320, generator=g))
    xd = x.to("cuda:0", dtype).contiguous(memory_format=torch.channels_last)
    y = torch.empty_like(xd)
    ret = torch.ops.fast_kernel.group_norm_fp16(xd, y, 1e-5, 32, "silu", w.to("cuda:0", dtype), b.to("cuda:0", dtype), True, False)
    torch.cuda.synchronize()
    assert ret is None and y.dtype == dtype and y.is_contiguous(memory_format=torch.channels_last)
    ref = O.group_norm(x, 32, w, b, 1e-5, "silu")
    assert_close_rel(y, ref, 2e-2, "fast_kernel.group_norm_fp16")
    # NCHW memory with the flag set, no affine, no activation
    xc = x.to("cuda:0", dtype).contiguous()
    yc = torch.empty_like(xc)
    torch.ops.fast_kernel.group_norm_fp16(xc, yc, 1e-6, 32, "none", w.to("cuda:0", dtype), b.to("cuda:0", dtype), False, True)
    assert_close_rel(yc, O.group_norm(x, 32, None, None, 1e-6), 2e-2, "fast_kernel.group_norm_fp16 nchw")
    with pytest.raises(RuntimeError):    # the reference only prints here (group_norm.cu:219-221)
        torch.ops.fast_kernel.group_norm_fp16(xd, y, 1e-5, 32, "relu", w.to("cuda:0", dtype), b.to("cuda:0", dtype), True, False)


@pytest.mark.gpu
def test_group_norm_fp16_serves_shapes_beyond_the_static_scratch():
    """More partial sums than the library's per-GPU array holds (here 1100 samples x 32 groups: 275 KiB against 256):
    the reference's op has no such limit, so the drop-in goes through the workspace form instead of refusing."""
    import katz_amd.fast_kernel_shim as shim
    from katz_amd import _lib
    from oracle import ops as O

    shim.install()
    print("fast_kernel.group_norm_fp16 N=1100", flush=True)
    assert _lib.load().kh_group_norm_workspace_bytes(1100, 64, 4, 32, 1) > 256 * 1024
    g = torch.Generator().manual_seed(5)
    x = bf16_round(torch.randn(1100, 64, 2, 2, generator=g) + 0.2)
    w, b = bf16_round(1 + 0.1 * torch.randn(64, generator=g)), bf16_round(0.1 * torch.randn(64, generator=g))
    xd = x.to("cuda:0", BF).contiguous(memory_format=torch.channels_last)
    y = torch.empty_like(xd)
    torch.ops.fast_kernel.group_norm_fp16(xd, y, 1e-5, 32, "silu", w.to("cuda:0", BF), b.to("cuda:0", BF), True, False)
    torch.cuda.synchronize()
    assert_close_rel(y, O.group_norm(x, 32, w, b, 1e-5, "silu"), 2e-2, "fast_kernel.group_norm_fp16 beyond the scratch")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fast_gelu_mul_fp16_reference_call(dtype):
    """activations.py:145: fast_gelu_mul_fp16(proj_2(h), proj_1(h)) = gelu_tanh(x) * m, callee-allocated."""
    import katz_amd.fast_kernel_shim as shim
    from oracle import ops as O

    shim.install()
    print("fast_kernel.fast_gelu_mul_fp16", dtype, flush=True)
    g = torch.Generator().manual_seed(4)
    x, m = bf16_round(torch.randn(2, 77, 1280, generator=g) * 2), bf16_round(torch.randn(2, 77, 1280, generator=g))
    if dtype == torch.float16:
        x, m = x.half().float(), m.half().float()
    out = torch.ops.fast_kernel.fast_gelu_mul_fp16(x.to("cuda:0", dtype), m.to("cuda:0", dtype))
    torch.cuda.synchronize()
    assert out.dtype == dtype and out.shape == x.shape
    assert_close_rel(out, O.gelu_mul(x, m, "tanh"), 2e-2, "fast_kernel.fast_gelu_mul_fp16")
    with pytest.raises(RuntimeError):    # gelu.cuh:45
        torch.ops.fast_kernel.fast_gelu_mul_fp16(x.to("cuda:0", dtype), m.to("cuda:0", dtype)[:, :5])
    with pytest.raises(RuntimeError):    # gelu.cuh:46
        torch.ops.fast_kernel.fast_gelu_mul_fp16(x.to("cuda:0", dtype).transpose(0, 1), m.to("cuda:0", dtype).transpose(0, 1))
