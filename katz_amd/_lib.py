"""ctypes binding of libkatz_hip.so (the C ABI declared in include/katz_hip.h).

There is no fallback: if the library is missing the import of any op fails with an error that says
how to build it.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libkatz_hip.so"

_P = c_void_p
_I = c_int64

# name -> (restype, argtypes); mirrors include/katz_hip.h one to one
SIGNATURES = {
    "kh_version": (c_int, []),
    "kh_error_string": (c_char_p, [c_int]),
    "kh_profile_begin": (c_int, []),
    "kh_profile_end": (c_int, [_P, _P, c_int]),
    "kh_lora_linear_bf16": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, c_int, _P]),
    "kh_lora_shrink_bf16": (c_int, [_P, _P, _P, _P, _I, _I, _I, _P]),
    "kh_lora_linear_pre_bf16": (c_int, [_P, _P, _P, _P, _I, _I, _P, _P, _P, _I, _I, _I, _I, c_int, _P]),
    "kh_lora_linear_grouped_bf16": (c_int, [_P, _P, _I, _I, _I, _I, _I, _I, c_int, _P]),
    "kh_lora_merge_grouped_bf16": (c_int, [_P, _P, _P, _I, _I, _I, c_float, c_int, _P]),
    "kh_lora_linear_f32": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P]),
    "kh_sgmv_shrink_bf16": (c_int, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P]),
    "kh_sgmv_expand_bf16": (c_int, [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P]),
    "kh_sgmv_fused_bf16": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "kh_sgmv_fused_grouped_bf16": (c_int, [_P, _P, _I, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "kh_attention_bf16": (c_int, [_P, _P, _P, _P] + [_I] * 13 + [c_float, _P]),
    "kh_group_norm_workspace_bytes": (c_int64, [_I, _I, _I, _I, c_int]),
    "kh_group_norm_bf16": (c_int, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, c_float, c_int, c_int, _P]),
    "kh_group_norm_static_bf16": (c_int, [_P, _P, _P, _P, _P, _I, _I, _I, _I, c_float, c_int, c_int, _P]),
    "kh_lora_linear_split_bf16": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, c_int, _P]),
    "kh_lora_linear_norm_bf16": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, c_float, _P,
                                         _I, _I, _I, _I, _I, c_int, _P]),
    "kh_lora_linear_xattn_bf16": (c_int, [_P] * 8 + [_P] * 5 + [c_float] + [_P] * 3 + [_I] * 11 + [c_float, c_int, _P]),
    "kh_lora_linear_xattn_ok": (c_int, [_I] * 6),
    "kh_lora_split_timeouts": (c_int, [_P, c_int]),
    "kh_set_weight_prefetch": (c_int, [_P, _I]),
    "kh_lora_linear_split_launches": (c_int, [_I, _I, _I, _I, _I, c_int]),
    "kh_layer_norm_bf16": (c_int, [_P, _P, _P, _P, _I, _I, c_float, _P]),
    "kh_geglu_bf16": (c_int, [_P, _P, _I, _I, c_int, _P]),
    "kh_gelu_mul_bf16": (c_int, [_P, _P, _P, _I, c_int, _P]),
    "kh_residual_add_bf16": (c_int, [_P, _P, c_int, c_float, _I, _P]),
    "kh_concat_residual_bf16": (c_int, [_P, _P, _P, c_int, c_float, _P, _I, _I, _I, _P]),
    "kh_upsample_nearest2x_nhwc_bf16": (c_int, [_P, _P, _I, _I, _I, _I, _P]),
    "kh_cfg_euler_step_bf16": (c_int, [_P, _P, _P, _P, _I, c_float, _P, c_int, _P]),
    "kh_conv_out_cfg_euler_bf16": (c_int, [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, c_float, _P, c_int, _P]),
    "kh_conv3x3_nhwc_bf16": (c_int, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P]),
    "kh_conv3x3_gn_splits": (_I, [_I] * 7),
    "kh_conv3x3_gn_stats_nhwc_bf16": (c_int, [_P] * 7 + [_I] * 7 + [_P]),
    "kh_group_norm_apply_bf16": (c_int, [_P] * 6 + [_I] * 5 + [c_float, c_int, _P]),
}

_lib = None


class KatzHipError(RuntimeError):
    """A katz_hip entry point rejected its arguments or the launch failed."""


def load() -> ctypes.CDLL:
    """Load libkatz_hip.so once and attach the prototypes. Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise KatzHipError(
            f"{LIB_PATH} is missing: build the HIP kernels with `python -m katz_amd.build` "
            "(needs hipcc); there is no CPU fallback for these ops"
        )
    # torch first: its HIP runtime must be the one this process initialises.  If libkatz_hip.so pulls in
    # a HIP runtime of its own before torch is imported, launches fail with hipErrorNoDevice.
    import torch  # noqa: F401

    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here means header and library disagree
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def is_loaded() -> bool:
    """True once load() has succeeded in this process (for code that must not trigger the load itself)."""
    return _lib is not None


def check(code: int, what: str) -> None:
    if code != 0:
        msg = load().kh_error_string(int(code)).decode()
        raise KatzHipError(f"{what} failed with code {code}: {msg}")
