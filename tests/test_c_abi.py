"""The C-ABI library loads without a GPU and exports exactly what include/katz_hip.h declares."""
import ctypes
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "katz_hip.h"


def declared_symbols():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(kh_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    syms = declared_symbols()
    for must in ("kh_lora_linear_bf16", "kh_lora_linear_f32", "kh_lora_shrink_bf16", "kh_lora_linear_pre_bf16",
                 "kh_sgmv_shrink_bf16", "kh_sgmv_expand_bf16", "kh_attention_bf16", "kh_group_norm_bf16",
                 "kh_layer_norm_bf16", "kh_geglu_bf16", "kh_gelu_mul_bf16", "kh_residual_add_bf16",
                 "kh_concat_residual_bf16", "kh_upsample_nearest2x_nhwc_bf16", "kh_version", "kh_error_string"):
        assert must in syms


def test_library_exports_every_declared_symbol():
    from katz_amd import _lib

    if not _lib.LIB_PATH.exists():
        pytest.skip("libkatz_hip.so not built (run python -m katz_amd.build)")
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} is declared in katz_hip.h but not exported"
    # the ctypes prototype table covers the header one to one
    assert sorted(_lib.SIGNATURES) == declared_symbols()


def test_argument_validation_needs_no_gpu():
    """Entry points reject bad arguments before touching the device."""
    from katz_amd import _lib

    if not _lib.LIB_PATH.exists():
        pytest.skip("libkatz_hip.so not built")
    lib = _lib.load()
    assert lib.kh_version() >= 1
    assert b"aligned" in lib.kh_error_string(-3)
    assert lib.kh_lora_linear_bf16(None, None, None, None, None, None, None, None, 1, 8, 8, 0, 0, None) == -1
    assert lib.kh_lora_linear_bf16(16, 16, None, None, None, None, None, 16, 4, 8, 12, 0, 0, None) == -2   # K % 8
    assert lib.kh_lora_linear_bf16(16, 16, None, 16, 16, 16, None, 16, 4, 8, 8, 160, 0, None) == -4        # R > 128
    assert lib.kh_lora_linear_bf16(8, 16, None, None, None, None, None, 16, 4, 8, 8, 0, 0, None) == -3     # alignment
    assert lib.kh_attention_bf16(16, 16, 16, 16, 1, 1, 4, 4, 32, 64, 64, 64, 64, 256, 256, 256, 256, 0.1, None) == -2
    assert lib.kh_group_norm_workspace_bytes(2, 320, 16384, 32, 1) > 0
    assert lib.kh_group_norm_workspace_bytes(2, 30, 64, 4, 1) == -1   # C % G != 0
    assert lib.kh_layer_norm_bf16(16, 16, None, None, 4, 4096, 1e-5, None) == -2  # D > 2048
    assert lib.kh_lora_shrink_bf16(16, 16, 16, 16, 4, 72, 32, None) == -2        # K % 64
    # the query projection with the text cross-attention in its epilogue
    assert lib.kh_lora_linear_xattn_ok(2048, 1280, 1280, 128, 1024, 77) == 1
    assert lib.kh_lora_linear_xattn_ok(2048, 1280, 1280, 128, 1024, 128) == 0      # more than 96 keys
    assert lib.kh_lora_linear_xattn_ok(2048, 1280, 1280, 128, 1000, 77) == 0       # T % 128
    assert lib.kh_lora_linear_xattn_bf16(*([None] * 13), 1e-5, *([None] * 3), 2048, 1280, 1280, 128, 1024, 77,
                                         1280, 1280, 1280, 98560, 98560, 0.125, 0, None) == -1
    assert lib.kh_lora_linear_xattn_bf16(*([16] * 13), 1e-5, *([16] * 3), 2048, 1280, 1280, 128, 1024, 128,
                                         1280, 1280, 1280, 163840, 163840, 0.125, 0, None) == -1
    # convolution with the next GroupNorm's statistics, and the norm's apply pass on them
    assert lib.kh_conv3x3_gn_splits(2, 32, 32, 1280, 1280, 1, 32) == 16
    assert lib.kh_conv3x3_gn_splits(2, 64, 64, 640, 640, 1, 32) == 32
    assert lib.kh_conv3x3_gn_splits(2, 32, 32, 1280, 1280, 1, 7) == 0              # groups do not divide the channels
    assert lib.kh_conv3x3_gn_splits(2, 128, 128, 320, 4, 1, 2) == 0                # no 160-column tiles
    assert lib.kh_conv3x3_gn_stats_nhwc_bf16(*([None] * 7), 2, 32, 32, 1280, 1280, 1, 32, None) == -1
    assert lib.kh_conv3x3_gn_stats_nhwc_bf16(16, 16, None, None, None, 16, 16, 2, 32, 32, 1280, 1280, 1, 7, None) == -1
    assert lib.kh_group_norm_apply_bf16(None, None, None, None, None, None, 16, 2, 1280, 1024, 32, 1e-5, 1, None) == -1
    assert lib.kh_group_norm_apply_bf16(16, 16, None, None, None, 16, 16, 2, 1290, 1024, 32, 1e-5, 1, None) == -1
    # several layers' segmented shrink + expand in one launch: the table is required, shapes as for the single layer
    assert lib.kh_sgmv_fused_grouped_bf16(16, None, 4, 16, 16, 16, 16, 8, 77, 1280, 2048, 128, None) == -1
    assert lib.kh_sgmv_fused_grouped_bf16(16, 16, 4, 16, 16, 16, 16, 8, 77, 1280, 2048, 160, None) == -4     # RP > 128
    assert lib.kh_sgmv_fused_grouped_bf16(16, 16, 4, 16, 16, 16, 16, 8, 77, 1200, 2048, 128, None) == -2     # N % 128
    # the entry point that allocates nothing: its limit and its arguments are checked before the first device call
    assert lib.kh_group_norm_static_bf16(16, 16, None, None, None, 4096, 4096, 65536, 32, 1e-5, 0, 1, None) == -4
    assert lib.kh_group_norm_static_bf16(None, 16, None, None, None, 2, 320, 64, 32, 1e-5, 0, 1, None) == -1


def test_a_refused_call_drops_the_pending_weight_prefetch_hint():
    """kh_set_weight_prefetch queues up to three ranges for the next launch of the linear / convolution family (a fourth
    is refused).  A call of that family that refuses its arguments must not leave them pending for an unrelated later
    launch: afterwards three new ranges can be queued again.  No device call is made."""
    from katz_amd import _lib

    if not _lib.LIB_PATH.exists():
        pytest.skip("libkatz_hip.so not built")
    lib = _lib.load()
    refused = (
        lambda: lib.kh_lora_linear_bf16(None, None, None, None, None, None, None, None, 1, 8, 8, 0, 0, None),
        lambda: lib.kh_lora_linear_pre_bf16(*([None] * 3), None, 0, 0, *([None] * 3), 1, 8, 32, 32, 0, None),
        lambda: lib.kh_lora_linear_split_bf16(*([None] * 10), 1, 8, 64, 32, 0, 0, None),
        lambda: lib.kh_lora_linear_norm_bf16(*([None] * 15), 1e-5, None, 1, 8, 64, 0, 0, 0, None),
        lambda: lib.kh_conv3x3_nhwc_bf16(None, None, None, None, None, 1, 8, 8, 32, 8, 1, None),
        lambda: lib.kh_conv3x3_gn_stats_nhwc_bf16(*([None] * 7), 2, 32, 32, 1280, 1280, 1, 32, None),
    )
    assert lib.kh_set_weight_prefetch(None, 0) == 0
    for call in refused:
        for _ in range(3):
            assert lib.kh_set_weight_prefetch(4096, 1 << 20) == 0
        assert lib.kh_set_weight_prefetch(4096, 1 << 20) == -4          # three are pending
        assert call() < 0
        for _ in range(3):                                               # ... and gone after the refused call
            assert lib.kh_set_weight_prefetch(4096, 1 << 20) == 0
        assert lib.kh_set_weight_prefetch(None, 0) == 0
