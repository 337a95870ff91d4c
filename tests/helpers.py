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


# ---- deterministic tensors for the committed reference fixtures -----------------------------------------------
# tests/golden/make_unet_tiny_fixture.py (run once, in the build container, against the reference's own modules) and
# the tests that read its output must hold identical weights and inputs without storing them: every tensor is a
# function of its name and shape only.

def det_tensor(name: str, shape, std: float = 1.0, mean: float = 0.0) -> torch.Tensor:
    """fp32 tensor of the given shape, N(mean, std), from a numpy PCG64 stream seeded by crc32(name)."""
    import zlib

    import numpy as np

    rng = np.random.Generator(np.random.PCG64(zlib.crc32(name.encode())))
    n = 1
    for s in shape:
        n *= int(s)
    a = rng.standard_normal(n).astype(np.float32) * np.float32(std) + np.float32(mean)
    return torch.from_numpy(a).reshape(tuple(int(s) for s in shape))


def det_state_dict(shapes, prefix: str = ""):
    """{key: tensor} for a {key: shape} map: weights of >= 2 dims ~ N(0, 1/fan_in), norm scales ~ 1 + 0.1 N(0,1), every
    other 1-D tensor (biases) ~ 0.1 N(0,1).  A norm scale is a 1-D `weight` (GroupNorm / LayerNorm)."""
    out = {}
    for k, shape in shapes.items():
        shape = tuple(shape)
        if len(shape) >= 2:
            fan_in = 1
            for s in shape[1:]:
                fan_in *= s
            out[k] = det_tensor(prefix + k, shape, std=fan_in ** -0.5)
        elif k.endswith("weight"):
            out[k] = det_tensor(prefix + k, shape, std=0.1, mean=1.0)
        else:
            out[k] = det_tensor(prefix + k, shape, std=0.1)
    return out


FIXTURE_UNET = dict(block_out_channels=(64, 128, 256), transformer_layers_per_block=(1, 2, 3),
                    num_attention_heads=(1, 2, 4), cross_attention_dim=128, addition_time_embed_dim=32,
                    projection_class_embeddings_input_dim=64 + 6 * 32)


def fixture_unet_inputs(latent: int):
    """Inputs of the reference-fixture runs at a `latent` x `latent` resolution (batch 2, 7 context tokens)."""
    B = 2
    time_ids = torch.tensor([[8.0 * latent, 8.0 * latent, 0, 0, 8.0 * latent, 8.0 * latent],
                             [8.0 * latent, 6.0 * latent, 4, 8, 8.0 * latent, 8.0 * latent]])
    return dict(sample=det_tensor(f"in.sample.{latent}", (B, 4, latent, latent)),
                timestep=500.0,
                encoder_hidden_states=det_tensor("in.context", (B, 7, 128)),
                text_embeds=det_tensor("in.text_embeds", (B, 64)),
                time_ids=time_ids,
                controlnet_cond=det_tensor(f"in.cond.{latent}", (B, 3, 8 * latent, 8 * latent), std=0.3, mean=0.5))


def fixture_residuals(latent: int, std: float = 0.3):
    """9 down residuals + 1 mid residual with the skip shapes of the fixture UNet (unet_2d_condition.py:539-563 scaled)."""
    c = FIXTURE_UNET["block_out_channels"]
    H = latent
    shapes = [(c[0], H), (c[0], H), (c[0], H), (c[0], H // 2), (c[1], H // 2), (c[1], H // 2), (c[1], H // 4),
              (c[2], H // 4), (c[2], H // 4)]
    down = [det_tensor(f"in.res.{i}.{latent}", (2, ch, h, h), std=std) for i, (ch, h) in enumerate(shapes)]
    mid = det_tensor(f"in.res.mid.{latent}", (2, c[2], H // 4, H // 4), std=std)
    return down, mid
