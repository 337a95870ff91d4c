"""Shared parity helpers for the test-suite."""
import torch


def bf16_round(t: torch.Tensor) -> torch.Tensor:
    """fp32 tensor holding bf16-representable values."""
    return t.to(torch.bfloat16).to(torch.float32)


def assert_close_rel(got: torch.Tensor, ref: torch.Tensor, rel: float, what: str = "") -> float:
    """Elementwise |got-ref| <= rel * (|ref| + rms(ref)).  For bf16 kernels rel = 2e-2 (the per-layer
    tolerance of the parity contract); returns the worst ratio err / (|ref| + rms)."""
    got = got.detach().float().cpu()
    ref = ref.detach().float().cpu()
    assert got.shape == ref.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite values in the result"
    rms = ref.pow(2).mean().sqrt().clamp_min(1e-12)
    ratio = ((got - ref).abs() / (ref.abs() + rms)).max().item()
    assert ratio <= rel, f"{what}: worst relative error {ratio:.3e} > {rel:.1e}"
    return ratio
