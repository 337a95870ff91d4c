"""Structural pins of the oracle's SDXL UNet wiring (no reference KAT exists for the full model)."""
import json
from pathlib import Path

import pytest
import torch

from oracle import blocks as Bk
from oracle.unet_sdxl import UNet2DConditionModel, UNetConfig

GOLDEN = Path(__file__).resolve().parent / "golden" / "sdxl_lora_keys.json"


@pytest.fixture(scope="module")
def sdxl_meta():
    with torch.device("meta"):
        return UNet2DConditionModel(UNetConfig.sdxl())


def test_lora_linear_names_match_reference_fixture(sdxl_meta):
    """The 722 LoRA-able linears and their in/out sizes equal the reference's key-match fixture
    (lora_info_shm/TheLastBen_Papercut_SDXL_key_match_unet.json + shapes + alphas)."""
    keys = json.loads(GOLDEN.read_text())
    lin = sdxl_meta.lora_linears()
    assert len(keys) == 722
    assert {k + ".weight" for k in lin} == set(keys)
    for k, meta in keys.items():
        m = lin[k[: -len(".weight")]]
        r, fin = meta["down"]
        fout, r2 = meta["up"]
        assert (m.in_features, m.out_features) == (fin, fout) and r == r2 == 64 and meta["alpha"] == 20000.0


def test_state_dict_uses_katz_module_names(sdxl_meta):
    sd = sdxl_meta.state_dict()
    # names the Katz fork's load hooks produce (resnet.py:336-350, unet_2d_condition.py:521-529)
    assert "down_blocks.0.resnets.0.norm_silu1.0.weight" in sd
    assert "down_blocks.0.resnets.0.norm_silu2.0.bias" in sd
    assert "conv_norm_silu.0.weight" in sd
    assert "mid_block.attentions.0.transformer_blocks.9.ff.net.0.proj.weight" in sd
    assert sd["add_embedding.linear_1.weight"].shape == (1280, 2816)
    n_params = sum(v.numel() for v in sd.values())
    assert abs(n_params - 2.567e9) < 0.01e9  # SDXL base UNet: ~2.57 B parameters


def test_tiny_unet_forward_shapes_and_skip_order():
    """Skip tensors follow the order / shapes of unet_2d_condition.py:539-563 (scaled to the tiny config),
    zero ControlNet residuals equal no ControlNet (the reference feeds zeros, pipeline_..._katz.py:1493-1505)."""
    torch.manual_seed(0)
    cfg = UNetConfig.tiny()
    m = UNet2DConditionModel(cfg).eval()
    B, H = 2, 16
    x = torch.randn(B, 4, H, H)
    ctx = torch.randn(B, 7, cfg.cross_attention_dim)
    added = dict(text_embeds=torch.randn(B, 64), time_ids=torch.tensor([[H * 8, H * 8, 0, 0, H * 8, H * 8]] * B).float())
    with torch.no_grad():
        skips, mid = m(x, 500, ctx, added, return_skips=True)
        c = cfg.block_out_channels
        exp = [(c[0], H), (c[0], H), (c[0], H), (c[0], H // 2), (c[1], H // 2), (c[1], H // 2), (c[1], H // 4),
               (c[2], H // 4), (c[2], H // 4)]
        assert [(s.shape[1], s.shape[2]) for s in skips] == exp
        assert mid.shape == (B, c[2], H // 4, H // 4)
        y0 = m(x, 500, ctx, added)
        y1 = m(x, 500, ctx, added, [torch.zeros_like(s) for s in skips], torch.zeros_like(mid))
        y2 = m(x, 500, ctx, added, [0.1 * torch.randn_like(s) for s in skips], 0.1 * torch.randn_like(mid))
    assert y0.shape == (B, 4, H, H)
    assert torch.equal(y0, y1)
    assert not torch.allclose(y0, y2)


# ---- numerical pin of the wiring: the reference's own UNet2DConditionModel on a tiny SDXL-topology configuration ----
FIXTURE = Path(__file__).resolve().parent / "golden" / "unet_tiny_reference.safetensors"


def _fixture_unet():
    from helpers import FIXTURE_UNET, det_state_dict

    m = UNet2DConditionModel(UNetConfig(**FIXTURE_UNET)).eval()
    m.load_state_dict(det_state_dict({k: v.shape for k, v in m.state_dict().items()}, "unet."))
    return m


def test_unet_forward_matches_reference_fixture():
    """oracle.unet_sdxl.UNet2DConditionModel.forward == the reference's forward (unet_2d_condition.py:1955-2075,
    residual run through :1127-1341) on identical weights and inputs, <= 1e-4.  The fixture was written by
    tests/golden/make_unet_tiny_fixture.py from the reference's modules; depths (1, 2, 3), two different time_ids
    rows and three distinct same-shape skips make transposed wiring (skip order, text/time concat order, embedding
    flip / shift, emb + aug_emb) change the output."""
    from safetensors.torch import load_file

    from helpers import fixture_residuals, fixture_unet_inputs

    gold = load_file(str(FIXTURE))
    m = _fixture_unet()
    i = fixture_unet_inputs(16)
    added = dict(text_embeds=i["text_embeds"], time_ids=i["time_ids"])
    down, mid = fixture_residuals(16)
    with torch.no_grad():
        y0 = m(i["sample"], i["timestep"], i["encoder_hidden_states"], added)
        y1 = m(i["sample"], i["timestep"], i["encoder_hidden_states"], added, down, mid)
        y_mid_only = m(i["sample"], i["timestep"], i["encoder_hidden_states"], added, None, mid)
    assert (y0 - gold["unet.out_plain"]).abs().max().item() <= 1e-4
    assert (y1 - gold["unet.out_residuals"]).abs().max().item() <= 1e-4
    # the residuals matter at this tolerance, so the comparison above is not vacuous
    assert (gold["unet.out_plain"] - gold["unet.out_residuals"]).abs().max().item() > 1e-2
    # the reference's eager forward (graphs off) applies the mid residual only (unet_2d_condition.py:1886-1898)
    assert (y_mid_only - gold["unet.out_residuals_eager"]).abs().max().item() <= 1e-4


def test_unet_fixture_detects_wiring_mistakes():
    """Each plausible wiring mistake moves the output by far more than the 1e-4 tolerance of the pin."""
    from safetensors.torch import load_file

    from helpers import fixture_residuals, fixture_unet_inputs

    gold = load_file(str(FIXTURE))
    m = _fixture_unet()
    i = fixture_unet_inputs(16)
    added = dict(text_embeds=i["text_embeds"], time_ids=i["time_ids"])
    down, mid = fixture_residuals(16)
    with torch.no_grad():
        swapped = list(down)
        swapped[1], swapped[2] = swapped[2], swapped[1]          # two of the three same-shape skips
        y = m(i["sample"], i["timestep"], i["encoder_hidden_states"], added, swapped, mid)
        assert (y - gold["unet.out_residuals"]).abs().max().item() > 1e-2
        ids = i["time_ids"][:, [1, 0, 2, 3, 4, 5]]               # order of the size conditioning
        y = m(i["sample"], i["timestep"], i["encoder_hidden_states"], dict(text_embeds=i["text_embeds"], time_ids=ids))
        assert (y - gold["unet.out_plain"]).abs().max().item() > 1e-3
        y = m(i["sample"], 499.0, i["encoder_hidden_states"], added)
        assert (y - gold["unet.out_plain"]).abs().max().item() > 1e-4
