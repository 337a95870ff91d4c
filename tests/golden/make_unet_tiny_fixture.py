"""Writes tests/golden/unet_tiny_reference.safetensors: outputs of the REFERENCE's own UNet2DConditionModel and
ControlNetModel on a tiny SDXL-topology configuration, for pinning the wiring of oracle/unet_sdxl.py and
oracle/controlnet.py numerically.

Run once, in the build container only (python tests/golden/make_unet_tiny_fixture.py): it imports the reference's
modules from /root/reference/diffusers-hf/src (diffusers/models/unets/unet_2d_condition.py:190-530, :1127-1341,
:1955-2075; diffusers/models/controlnet.py:201-466, :687-847).  Nothing of the reference is copied: the fixture holds
output tensors only.  Weights and inputs are not stored either; both sides rebuild them from tests/helpers.py
(det_state_dict / fixture_unet_inputs / fixture_residuals: functions of tensor name and shape).

What the import needs here: `fast_kernel` (the CUDA extension, imported unconditionally by models/normalization.py:23
and models/activations.py:21 but only called when ENABLE_FUSED_NORM_SILU / ENABLE_FUSED_GEGLU are set) is an empty
module, and `huggingface_hub.cached_download` (removed upstream, imported by utils/dynamic_modules_utils.py:28) is a
None attribute; the four ENABLE_* flags are unset so the model runs the plain torch modules.  peft is absent, which
these two forwards do not need.

The residual run calls _down_forward + _up_forward (unet_2d_condition.py:1127-1341), the body the reference runs under
its graphs in every Katz configuration: it adds all nine skip residuals and the mid residual.  (The eager forward,
:1886-1898, applies the nine only when `down_intrablock_additional_residuals` is given; the fixture records that
output too, as `unet.out_residuals_eager`, to document the difference.)
"""
import json
import os
import sys
import types
from pathlib import Path

HERE = Path(__file__).resolve().parent
REFERENCE_SRC = Path("/root/reference/diffusers-hf/src")
OUT = HERE / "unet_tiny_reference.safetensors"


def main():
    for k in ("ENABLE_CUDA_GRAPH", "ENABLE_FUSED_GEGLU", "ENABLE_FUSED_NORM_SILU", "ENABLE_CHANNELS_LAST"):
        os.environ.pop(k, None)
    sys.modules["fast_kernel"] = types.ModuleType("fast_kernel")
    import huggingface_hub

    if not hasattr(huggingface_hub, "cached_download"):
        huggingface_hub.cached_download = None
    sys.path.insert(0, str(REFERENCE_SRC))
    sys.path.insert(0, str(HERE.parent))

    import torch
    from safetensors.torch import save_file

    from diffusers.models.controlnet import ControlNetModel
    from diffusers.models.unets.unet_2d_condition import UNet2DConditionModel
    from helpers import FIXTURE_UNET, det_state_dict, fixture_residuals, fixture_unet_inputs

    torch.manual_seed(0)
    cfg = FIXTURE_UNET
    unet = UNet2DConditionModel(
        sample_size=16, in_channels=4, out_channels=4,
        down_block_types=("DownBlock2D", "CrossAttnDownBlock2D", "CrossAttnDownBlock2D"),
        up_block_types=("CrossAttnUpBlock2D", "CrossAttnUpBlock2D", "UpBlock2D"),
        block_out_channels=cfg["block_out_channels"], layers_per_block=2,
        cross_attention_dim=cfg["cross_attention_dim"],
        transformer_layers_per_block=cfg["transformer_layers_per_block"],
        attention_head_dim=cfg["num_attention_heads"],   # SDXL's config stores the head COUNT under this name
        use_linear_projection=True, addition_embed_type="text_time",
        addition_time_embed_dim=cfg["addition_time_embed_dim"],
        projection_class_embeddings_input_dim=cfg["projection_class_embeddings_input_dim"], norm_num_groups=32,
    ).eval()
    unet.load_state_dict(det_state_dict({k: v.shape for k, v in unet.state_dict().items()}, "unet."))
    controlnet = ControlNetModel.from_unet(unet).eval()
    controlnet.load_state_dict(det_state_dict({k: v.shape for k, v in controlnet.state_dict().items()}, "controlnet."))

    out = {}
    with torch.no_grad():
        # ---- UNet at 16x16 latents
        i = fixture_unet_inputs(16)
        added = dict(text_embeds=i["text_embeds"], time_ids=i["time_ids"])
        t = torch.tensor(i["timestep"])
        out["unet.out_plain"] = unet(i["sample"], t, i["encoder_hidden_states"], added_cond_kwargs=added,
                                     return_dict=False)[0]
        down, mid = fixture_residuals(16)
        sample, emb, skips, ehs = unet._down_forward(i["sample"], t, i["encoder_hidden_states"],
                                                     added_cond_kwargs=added)
        out["unet.out_residuals"] = unet._up_forward(sample, emb, skips, tuple(down), mid, ehs, None, None, None,
                                                     return_dict=False)[0]
        out["unet.out_residuals_eager"] = unet(i["sample"], t, i["encoder_hidden_states"], added_cond_kwargs=added,
                                               down_block_additional_residuals=tuple(down),
                                               mid_block_additional_residual=mid, return_dict=False)[0]
        # ---- ControlNet at 8x8 latents (64x64 conditioning image), non-zero "zero" convolutions, Katz's default scale
        i = fixture_unet_inputs(8)
        added = dict(text_embeds=i["text_embeds"], time_ids=i["time_ids"])
        d, m = controlnet(i["sample"], t, i["encoder_hidden_states"], i["controlnet_cond"],
                          added_cond_kwargs=added)       # conditioning_scale: the fork's default, 0.5
        assert len(d) == 9
        for j, r in enumerate(d):
            out[f"controlnet.down.{j}"] = r
        out["controlnet.mid"] = m
        out["controlnet.mid_scale1"] = controlnet(i["sample"], t, i["encoder_hidden_states"], i["controlnet_cond"],
                                                  conditioning_scale=1.0, added_cond_kwargs=added)[1]
    out = {k: v.detach().float().contiguous() for k, v in out.items()}
    meta = {"config": json.dumps({k: list(v) if isinstance(v, tuple) else v for k, v in cfg.items()}),
            "made_by": "tests/golden/make_unet_tiny_fixture.py",
            "torch": torch.__version__,
            "n_unet_tensors": str(len(unet.state_dict())), "n_controlnet_tensors": str(len(controlnet.state_dict()))}
    save_file(out, str(OUT), metadata=meta)
    for k, v in out.items():
        print(f"{k:34s} {tuple(v.shape)}  rms {v.pow(2).mean().sqrt().item():.4f}")
    print("wrote", OUT, OUT.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
