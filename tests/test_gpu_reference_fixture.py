"""The product UNet / ControlNet (katz_amd on the HIP kernels, bf16) against outputs of the REFERENCE's own modules.

tests/golden/unet_tiny_reference.safetensors holds what the reference's UNet2DConditionModel and ControlNetModel
return on a tiny SDXL-topology configuration (written in the build container by tests/golden/make_unet_tiny_fixture.py;
weights and inputs are functions of tensor names, tests/helpers.py).  The reference ran in fp32 on unrounded weights,
the product rounds weights and every layer's output to bf16: the gate is BASELINE's whole-model one, cosine >= 0.999.
"""
from pathlib import Path

import pytest
import torch
from safetensors.torch import load_file

from helpers import (FIXTURE_UNET, assert_close_rel, cosine, det_state_dict, fixture_residuals, fixture_unet_inputs)

pytestmark = pytest.mark.gpu
BF = torch.bfloat16
DEV = "cuda:0"
GOLD = Path(__file__).resolve().parent / "golden" / "unet_tiny_reference.safetensors"


def _build(cls_name, prefix):
    import katz_amd.layers as L
    from katz_amd.controlnet import ControlNetModel
    from katz_amd.unet_2d_condition import UNet2DConditionModel, UNetConfig

    L.SKIP_INIT = True
    try:
        m = {"unet": UNet2DConditionModel, "controlnet": ControlNetModel}[cls_name](UNetConfig(**FIXTURE_UNET))
    finally:
        L.SKIP_INIT = False
    m.load_state_dict(det_state_dict({k: v.shape for k, v in m.state_dict().items()}, prefix), strict=True)
    return m.to_runtime(DEV, BF)


def test_unet_step_matches_reference_outputs():
    print("unet vs reference fixture", flush=True)
    gold = load_file(str(GOLD))
    unet = _build("unet", "unet.")
    i = fixture_unet_inputs(16)
    added = {"text_embeds": i["text_embeds"].to(DEV), "time_ids": i["time_ids"].to(DEV)}
    down, mid = fixture_residuals(16)
    t = torch.tensor([i["timestep"]], device=DEV)
    with torch.no_grad():
        y0 = unet(i["sample"].to(DEV), t, i["encoder_hidden_states"].to(DEV), added_cond_kwargs=added).sample
        y1 = unet(i["sample"].to(DEV), t, i["encoder_hidden_states"].to(DEV), added_cond_kwargs=added,
                  down_block_additional_residuals=[d.to(DEV) for d in down],
                  mid_block_additional_residual=mid.to(DEV)).sample
    torch.cuda.synchronize()
    c0, c1 = cosine(y0, gold["unet.out_plain"]), cosine(y1, gold["unet.out_residuals"])
    print(f"cosine plain {c0:.6f} residuals {c1:.6f}", flush=True)
    assert c0 >= 0.999 and c1 >= 0.999, (c0, c1)
    assert_close_rel(y1, gold["unet.out_residuals"], 1e-1, "unet vs reference")
    # all ten residuals are applied (the reference's graph path), not the mid one alone (its eager path)
    assert cosine(y1, gold["unet.out_residuals"]) > cosine(y1, gold["unet.out_residuals_eager"])


def test_controlnet_matches_reference_outputs():
    print("controlnet vs reference fixture", flush=True)
    gold = load_file(str(GOLD))
    cn = _build("controlnet", "controlnet.")
    i = fixture_unet_inputs(8)
    added = {"text_embeds": i["text_embeds"].to(DEV), "time_ids": i["time_ids"].to(DEV)}
    t = torch.tensor([i["timestep"]], device=DEV)
    with torch.no_grad():
        down, mid = cn(i["sample"].to(DEV), t, i["encoder_hidden_states"].to(DEV), i["controlnet_cond"].to(DEV),
                       added_cond_kwargs=added)
    torch.cuda.synchronize()
    assert len(down) == 9
    for j, (g, r) in enumerate(zip(list(down) + [mid], [gold[f"controlnet.down.{k}"] for k in range(9)] + [gold["controlnet.mid"]])):
        c = cosine(g, r)
        print(f"residual {j}: cosine {c:.6f}", flush=True)
        assert g.shape == r.shape and c >= 0.999, (j, c)
