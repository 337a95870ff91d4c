"""Structure and closed-form checks of the oracle ControlNet (tiny configuration, CPU, seconds)."""
import torch

from oracle.controlnet import ControlNetModel
from oracle.unet_sdxl import UNet2DConditionModel, UNetConfig


def _inputs(cfg, hw=16, seed=0):
    g = torch.Generator().manual_seed(seed)
    sample = torch.randn(2, cfg.in_channels, hw, hw, generator=g)
    ctx = torch.randn(2, 7, cfg.cross_attention_dim, generator=g)
    added = {"text_embeds": torch.randn(2, cfg.projection_class_embeddings_input_dim - 6 * cfg.addition_time_embed_dim, generator=g),
             "time_ids": torch.tensor([[hw * 8, hw * 8, 0, 0, hw * 8, hw * 8]] * 2, dtype=torch.float32)}
    cond = torch.rand(2, 3, hw * 8, hw * 8, generator=g)
    return sample, ctx, added, cond


def test_fresh_controlnet_outputs_exact_zeros_with_reference_shapes():
    cfg = UNetConfig.tiny()
    torch.manual_seed(0)
    cn = ControlNetModel(cfg).eval()
    sample, ctx, added, cond = _inputs(cfg)
    with torch.no_grad():
        down, mid = cn(sample, 500.0, ctx, cond, 0.5, added)
    boc = cfg.block_out_channels
    # the reference's placeholder shapes (unet_2d_condition.py:539-563) at this latent size
    expect = [(boc[0], 16)] * 3 + [(boc[0], 8), (boc[1], 8), (boc[1], 8), (boc[1], 4), (boc[2], 4), (boc[2], 4)]
    assert [(d.shape[1], d.shape[2]) for d in down] == expect and mid.shape == (2, boc[2], 4, 4)
    assert all(torch.count_nonzero(d) == 0 for d in down) and torch.count_nonzero(mid) == 0
    assert len(cn.controlnet_down_blocks) == 9


def test_identity_zero_convs_reproduce_the_unet_encoder():
    """ControlNet.from_unet copies the UNet encoder; with a zero conditioning embedding (its conv_out is
    zero-initialised) and identity 1x1 convs the residuals are conditioning_scale x the UNet's skips."""
    cfg = UNetConfig.tiny()
    torch.manual_seed(1)
    unet = UNet2DConditionModel(cfg).eval()
    cn = ControlNetModel(cfg).eval()
    sd = unet.state_dict()
    own = cn.state_dict()
    cn.load_state_dict({k: (sd[k] if k in sd else v) for k, v in own.items()})
    with torch.no_grad():
        for zc in list(cn.controlnet_down_blocks) + [cn.controlnet_mid_block]:
            zc.weight.copy_(torch.eye(zc.weight.shape[0]).reshape(zc.weight.shape))
        sample, ctx, added, cond = _inputs(cfg, seed=2)
        down, mid = cn(sample, 300.0, ctx, cond, 0.5, added)
        skips, mid_ref = unet(sample, 300.0, ctx, added, return_skips=True)
    for d, s in zip(down, skips):
        assert torch.allclose(d, s * 0.5, atol=1e-6)
    assert torch.allclose(mid, mid_ref * 0.5, atol=1e-6)


def test_conditioning_image_enters_after_conv_in():
    """With a non-zero embedding conv_out the conditioning changes every residual; scale is linear."""
    cfg = UNetConfig.tiny()
    torch.manual_seed(3)
    cn = ControlNetModel(cfg).eval()
    with torch.no_grad():
        torch.nn.init.normal_(cn.controlnet_cond_embedding.conv_out.weight, std=0.05)
        for zc in list(cn.controlnet_down_blocks) + [cn.controlnet_mid_block]:
            torch.nn.init.normal_(zc.weight, std=0.05)
        sample, ctx, added, cond = _inputs(cfg, seed=4)
        d1, m1 = cn(sample, 10.0, ctx, cond, 1.0, added)
        d2, m2 = cn(sample, 10.0, ctx, cond, 0.25, added)
        d3, _ = cn(sample, 10.0, ctx, torch.zeros_like(cond), 1.0, added)
    assert all(torch.allclose(a * 0.25, b, atol=1e-6) for a, b in zip(d1, d2)) and torch.allclose(m1 * 0.25, m2, atol=1e-6)
    assert not torch.allclose(d1[0], d3[0])
    # first residual = zero_conv0(conv_in(sample) + embedding(cond)) exactly
    e = cn.controlnet_cond_embedding(cond)
    assert e.shape == (2, cfg.block_out_channels[0], 16, 16)
    assert torch.allclose(d1[0], cn.controlnet_down_blocks[0](cn.conv_in(sample) + e), atol=1e-6)


def test_controlnet_forward_matches_reference_fixture():
    """oracle.controlnet.ControlNetModel.forward == the reference's ControlNetModel.forward (controlnet.py:687-847,
    built with from_unet :432-506) on identical weights (random, non-zero zero-convs and conditioning embedding) and
    inputs, <= 1e-4; default conditioning_scale 0.5 (:693) and 1.0.  Fixture: tests/golden/make_unet_tiny_fixture.py."""
    from pathlib import Path

    from safetensors.torch import load_file

    from helpers import FIXTURE_UNET, det_state_dict, fixture_unet_inputs

    gold = load_file(str(Path(__file__).resolve().parent / "golden" / "unet_tiny_reference.safetensors"))
    cn = ControlNetModel(UNetConfig(**FIXTURE_UNET)).eval()
    cn.load_state_dict(det_state_dict({k: v.shape for k, v in cn.state_dict().items()}, "controlnet."))
    i = fixture_unet_inputs(8)
    added = dict(text_embeds=i["text_embeds"], time_ids=i["time_ids"])
    with torch.no_grad():
        down, mid = cn(i["sample"], i["timestep"], i["encoder_hidden_states"], i["controlnet_cond"],
                       added_cond_kwargs=added)
        _, mid1 = cn(i["sample"], i["timestep"], i["encoder_hidden_states"], i["controlnet_cond"], 1.0, added)
    assert len(down) == 9
    for j, d in enumerate(down):
        ref = gold[f"controlnet.down.{j}"]
        assert d.shape == ref.shape
        assert (d - ref).abs().max().item() <= 1e-4 * max(1.0, ref.abs().max().item()), j
    assert (mid - gold["controlnet.mid"]).abs().max().item() <= 1e-4 * gold["controlnet.mid"].abs().max().item()
    assert (mid1 - gold["controlnet.mid_scale1"]).abs().max().item() <= 1e-4 * gold["controlnet.mid_scale1"].abs().max().item()
