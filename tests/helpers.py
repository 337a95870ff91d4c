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


def random_lora(linears, rank: int, seed: int, std: float = 0.02):
    """{module name: (down [r,in], up [out,r])} of bf16-representable fp32 values for a dict of linear
    modules (anything with in_features / out_features)."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, m in linears.items():
        out[name] = (bf16_round(torch.randn(rank, m.in_features, generator=g) * std),
                     bf16_round(torch.randn(m.out_features, rank, generator=g) * std))
    return out


def katz_lora_state_dict(tensors):
    """Spell a {module: (down, up)} dict with the converted-kohya keys the reference keeps in shared
    memory: attention projections under `<attn>.processor.to_q_lora.down.weight`, the rest under
    `<module>.lora.down.weight`, all prefixed `unet.`."""
    sd = {}
    for mod, (down, up) in tensors.items():
        head, _, leaf = mod.rpartition(".")
        if leaf in ("to_q", "to_k", "to_v"):
            base = f"unet.{head}.processor.{leaf}_lora"
        elif mod.endswith(".to_out.0"):
            base = f"unet.{mod[:-len('.to_out.0')]}.processor.to_out_lora"
        else:
            base = f"unet.{mod}.lora"
        sd[base + ".down.weight"] = down
        sd[base + ".up.weight"] = up
    return sd


def round_module_to_bf16_(module):
    """Round every parameter of an fp32 oracle module to bf16-representable values in place, so the
    product (bf16) and the oracle (fp32) hold identical weights."""
    with torch.no_grad():
        for p in module.parameters():
            p.copy_(bf16_round(p))
    return module


def cosine(a, b):
    a = a.detach().float().flatten().cpu()
    b = b.detach().float().flatten().cpu()
    return (torch.dot(a, b) / (a.norm() * b.norm()).clamp_min(1e-30)).item()
