"""Drop-in for the reference's native extension `fast_kernel`.

The reference imports `fast_kernel` unconditionally (diffusers-hf/src/diffusers/models/normalization.py:23,
activations.py:21); importing it loads `fast_kernel._C`, whose static initialiser registers two ops with
TORCH_LIBRARY(fast_kernel, m) (diffusers-hf/src/fast_kernel/fast_kernel/csrc/main.cpp:10-12, bind.cu:12-15):

    torch.ops.fast_kernel.group_norm_fp16(x, y, eps, num_groups, activation, weight, bias, affine, channels_last) -> ()
    torch.ops.fast_kernel.fast_gelu_mul_fp16(x, m) -> Tensor

`install()` registers the same two ops, same names, argument lists and error behaviour, on the katz_hip kernels, and
puts this module into sys.modules under the name `fast_kernel`, so the reference's `import fast_kernel` and its two
call sites (normalization.py:91, activations.py:145) work unchanged:

    import katz_amd.fast_kernel_shim as shim; shim.install()      # before `import diffusers`

Differences that a caller can see, all on the side of failing loudly:
  * an unknown activation raises (the reference prints and returns garbage, group_norm.cu:219-221);
  * a failed launch raises (the reference drops the cudaError_t, group_norm.cu:167-169);
  * the kernels compute on bf16 storage.  bf16 tensors are used as they are; fp16 tensors (the reference's
    GroupNorm.forward casts to fp16 before the call, normalization.py:88-90) are converted on the way in and out.
group_norm_fp16 allocates nothing on bf16 tensors (kh_group_norm_static_bf16 keeps its partial sums in a per-GPU array
of the library), so unlike the reference's op (two torch::empty per call, group_norm.cu:240-242) it can be captured.
Limits of that array, and what the shim does about them:
  * ONE array per GPU: calls that overlap on one GPU (two streams) race on it -- call the op from one stream per GPU;
  * its device address is looked up on the first call per device, which must not happen under capture: `install()`
    makes that call for the current device when a GPU is there; on another device run the op once eagerly first;
  * it holds 256 KiB of partial sums (about N <= 1024 samples at 32 groups, NHWC).  Larger shapes, which the reference's
    op serves, go through kh_group_norm_bf16 with a torch-allocated workspace instead (that path allocates on first use
    and when it grows: warm it up before capturing).
"""
from __future__ import annotations

import sys

import torch

from . import _lib

_registered = None   # the torch.library.Library object: it must stay alive for the ops to stay registered
BF16, FP16 = torch.bfloat16, torch.float16


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream   # at::cuda::getCurrentCUDAStream(), group_norm.cu:249, gelu.cuh:56


def _as_bf16(t: torch.Tensor) -> torch.Tensor:
    return t if t.dtype == BF16 else t.to(BF16)


def group_norm_fp16(x, y, eps, num_groups, activation, weight, bias, affine, channels_last):
    """y <- act(group_norm(x)) for a 4-D x.  The last flag is forwarded by the reference as `channels_first`
    (group_norm.cu:273 -> :233): False, what normalization.py:91 passes, means the memory is NHWC."""
    lib = _lib.load()
    if x.dim() != 4 or y.shape != x.shape or x.dtype not in (BF16, FP16) or y.dtype != x.dtype:
        raise RuntimeError("group_norm_fp16: x and y must be 4-D half / bfloat16 tensors of one shape and dtype")
    if activation not in ("none", "silu"):
        raise RuntimeError(f"group_norm_fp16: unsupported activation {activation!r}")
    n, c, h, w = x.shape
    nhwc = not channels_last
    fmt = torch.channels_last if nhwc else torch.contiguous_format
    if not x.is_contiguous(memory_format=fmt) or not y.is_contiguous(memory_format=fmt):
        raise RuntimeError("group_norm_fp16: x and y must be dense in the memory format the last argument names")
    xb = _as_bf16(x)
    yb = y if y.dtype == BF16 else torch.empty_like(xb)
    gamma = _as_bf16(weight) if affine else None
    beta = _as_bf16(bias) if affine else None
    rc = lib.kh_group_norm_static_bf16(xb.data_ptr(), yb.data_ptr(),
                                       None if gamma is None else gamma.data_ptr(),
                                       None if beta is None else beta.data_ptr(), None,
                                       n, c, h * w, int(num_groups), float(eps), 1 if activation == "silu" else 0,
                                       1 if nhwc else 0, _stream())
    if rc == -4:     # KH_ERR_TOO_LARGE: more partial sums than the library's per-GPU array holds
        from . import ops

        try:
            ops.group_norm(xb, int(num_groups), gamma, beta, float(eps), activation, out=yb)
        except (_lib.KatzHipError, ValueError, TypeError) as e:
            raise RuntimeError(f"group_norm_fp16: {e}") from e
    elif rc != 0:
        raise RuntimeError(f"group_norm_fp16: {lib.kh_error_string(int(rc)).decode()}")
    if yb is not y:
        y.copy_(yb)


def fast_gelu_mul_fp16(x, m):
    """gelu_tanh(x) * m, callee-allocated (gelu.cuh:29-59); same checks as the reference's TORCH_CHECKs (:45-47)."""
    lib = _lib.load()
    if x.shape != m.shape:
        raise RuntimeError("Input tensors x and m must have the same shape.")
    if not x.is_contiguous():
        raise RuntimeError("Input tensor x must be contiguous.")
    if not m.is_contiguous():
        raise RuntimeError("Input tensor m must be contiguous.")
    if x.dtype not in (BF16, FP16) or m.dtype != x.dtype:
        raise RuntimeError("fast_gelu_mul_fp16: x and m must be half / bfloat16 tensors of one dtype")
    xb, mb = _as_bf16(x), _as_bf16(m)
    out = torch.empty_like(xb)
    if x.numel():
        rc = lib.kh_gelu_mul_bf16(xb.data_ptr(), mb.data_ptr(), out.data_ptr(), x.numel(), 1, _stream())
        if rc != 0:
            raise RuntimeError(f"fast_gelu_mul_fp16: {lib.kh_error_string(int(rc)).decode()}")
    return out if x.dtype == BF16 else out.to(x.dtype)


def install() -> None:
    """Register torch.ops.fast_kernel.* (once per process) and make `import fast_kernel` resolve to this module."""
    global _registered
    if _registered is None:
        lib = torch.library.Library("fast_kernel", "DEF")
        lib.define("group_norm_fp16(Tensor x, Tensor(a!) y, float eps, int num_groups, str activation, "
                   "Tensor weight, Tensor bias, bool affine, bool channels_last) -> ()")
        lib.define("fast_gelu_mul_fp16(Tensor x, Tensor m) -> Tensor")
        lib.impl("group_norm_fp16", group_norm_fp16, "CUDA")
        lib.impl("fast_gelu_mul_fp16", fast_gelu_mul_fp16, "CUDA")
        _registered = lib
    sys.modules.setdefault("fast_kernel", sys.modules[__name__])
    if torch.cuda.is_available() and not torch.cuda.is_current_stream_capturing():
        # the first call per device resolves the address of the library's per-GPU array: do it here, outside any capture
        x = torch.zeros(1, 8, 2, 4, dtype=BF16, device="cuda")      # NCHW, 8 pixels: the smallest shape the kernels take
        group_norm_fp16(x, torch.empty_like(x), 1e-5, 1, "none", None, None, False, True)
