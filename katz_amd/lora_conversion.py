"""Kohya-format (sd-scripts / SGM naming) LoRA state dicts -> the key spelling the reference keeps after
conversion, which is what `UNet2DConditionModel.load_lora_into_unet` and Katz's shared-memory sidecars use.

Mirrors the effect of `_maybe_map_sgm_blocks_to_diffusers` and `_convert_kohya_lora_to_diffusers`
(diffusers-hf/src/diffusers/loaders/lora_conversion_utils.py:23-122, :126-287) for UNet keys:

    lora_unet_input_blocks_4_1_transformer_blocks_0_attn1_to_q.lora_down.weight
 -> unet.down_blocks.1.attentions.0.transformer_blocks.0.attn1.processor.to_q_lora.down.weight
    lora_unet_middle_block_1_proj_in.lora_up.weight
 -> unet.mid_block.attentions.0.proj_in.lora.up.weight
    lora_unet_output_blocks_2_1_transformer_blocks_3_ff_net_0_proj.alpha
 -> network_alphas["unet.up_blocks.0.attentions.2.transformer_blocks.3.ff.net.0.proj.alpha"]

    lora_unet_input_blocks_4_0_in_layers_2.lora_down.weight       (a resnet's first convolution)
 -> unet.down_blocks.1.resnets.0.conv1.lora.down.weight
    lora_unet_input_blocks_3_0_op / lora_unet_output_blocks_2_2_conv  (samplers)
 -> unet.down_blocks.0.downsamplers.0.conv / unet.up_blocks.0.upsamplers.0.conv

It is a small parser, not a chain of string replacements: the key is split into the block address (SGM
`input_blocks_i_j` / `middle_block_j` / `output_blocks_i_j`, or diffusers `down_blocks_b_attentions_l`) and the
module path inside the block.  Text-encoder entries (`lora_te*_`) are not on the UNet path: they are returned
untouched under `passthrough`.  Convolution targets are the resnets' conv1 / conv2 / conv_shortcut (SGM in_layers_2 /
out_layers_3 / skip_connection) and the sampler convolutions; the resnets' time_emb_proj (emb_layers_1) is refused.
"""
from __future__ import annotations

import re
from typing import Dict, Mapping, Tuple

import torch

_SUFFIXES = (".lora_down.weight", ".lora_up.weight", ".alpha")
_BLOCK_SGM = re.compile(r"^(input_blocks|output_blocks)_(\d+)_(\d+)_(.+)$")
_BLOCK_MID = re.compile(r"^middle_block_(\d+)_(.+)$")
_BLOCK_DIFF = re.compile(r"^(down_blocks|up_blocks)_(\d+)_attentions_(\d+)_(.+)$")
_BLOCK_DIFF_MID = re.compile(r"^mid_block_attentions_(\d+)_(.+)$")
_RESNET_INNER = {"in_layers_2": "conv1", "out_layers_3": "conv2", "skip_connection": "conv_shortcut",
                 "conv1": "conv1", "conv2": "conv2", "conv_shortcut": "conv_shortcut"}
_BLOCK_DIFF_RES = re.compile(r"^(down_blocks|up_blocks)_(\d+)_(resnets|downsamplers|upsamplers)_(\d+)_(.+)$")
_BLOCK_DIFF_MID_RES = re.compile(r"^mid_block_resnets_(\d+)_(.+)$")
_INNER = re.compile(r"^(proj_in|proj_out|transformer_blocks_(\d+)_(attn[12]_to_(?:q|k|v|out_0)|ff_net_0_proj|ff_net_2))$")


def _block_address(name: str, layers_per_block: int) -> Tuple[str, str]:
    """-> ('down_blocks.1.attentions.0' | 'down_blocks.1.resnets.0' | 'down_blocks.0.downsamplers.0' | ..., rest of
    the name).  SGM numbering (lora_conversion_utils.py:78-118): input block i >= 1 is layer (i-1) % 3 of down block
    (i-1) // 3, output block i layer i % 3 of up block i // 3 (for layers_per_block 2); inside a block, slot 0 is the
    resnet, 1 the transformer, 2 the upsampler, and a slot named `op` the downsampler."""
    m = _BLOCK_SGM.match(name)
    if m:
        kind, i, j, rest = m.group(1), int(m.group(2)), int(m.group(3)), m.group(4)
        per = layers_per_block + 1
        if kind == "input_blocks":
            if i < 1:
                raise ValueError(f"{name}: input block 0 is conv_in and holds no LoRA target")
            blk, layer = (i - 1) // per, (i - 1) % per
            if rest == "op":
                return f"down_blocks.{blk}.downsamplers.0", "conv"
            inner = {0: "resnets", 1: "attentions"}.get(j)
            if inner is None:
                raise ValueError(f"{name}: input blocks have slots 0 (resnet) and 1 (transformer)")
            return f"down_blocks.{blk}.{inner}.{layer}", rest
        blk, layer = i // per, i % per
        if j == 2:
            return f"up_blocks.{blk}.upsamplers.0", rest
        inner = {0: "resnets", 1: "attentions"}.get(j)
        if inner is None:
            raise ValueError(f"{name}: output blocks have slots 0 (resnet), 1 (transformer) and 2 (upsampler)")
        return f"up_blocks.{blk}.{inner}.{layer}", rest
    m = _BLOCK_MID.match(name)
    if m:
        slot = int(m.group(1))
        if slot not in (0, 1, 2):
            raise ValueError(f"{name}: invalid middle block id {slot}")
        return ("mid_block.attentions.0" if slot == 1 else f"mid_block.resnets.{slot // 2}"), m.group(2)
    m = _BLOCK_DIFF_RES.match(name)
    if m:
        return f"{m.group(1)}.{m.group(2)}.{m.group(3)}.{m.group(4)}", m.group(5)
    m = _BLOCK_DIFF_MID_RES.match(name)
    if m:
        return f"mid_block.resnets.{m.group(1)}", m.group(2)
    m = _BLOCK_DIFF.match(name)
    if m:
        return f"{m.group(1)}.{m.group(2)}.attentions.{m.group(3)}", m.group(4)
    m = _BLOCK_DIFF_MID.match(name)
    if m:
        return f"mid_block.attentions.{m.group(1)}", m.group(2)
    raise ValueError(f"unrecognised kohya UNet LoRA key {name!r}")


def _module_path(block: str, rest: str) -> Tuple[str, bool]:
    """-> (diffusers module path, is attention projection)."""
    if ".resnets." in block:
        if rest in ("emb_layers_1", "time_emb_proj"):
            raise NotImplementedError(f"{block}: LoRA on a resnet's time_emb_proj is not supported")
        if rest not in _RESNET_INNER:
            raise ValueError(f"{block}: unknown resnet LoRA target {rest!r}")
        return f"{block}.{_RESNET_INNER[rest]}", False
    if ".downsamplers." in block or ".upsamplers." in block:
        if rest not in ("conv", "op"):
            raise ValueError(f"{block}: unknown sampler LoRA target {rest!r}")
        return f"{block}.conv", False
    m = _INNER.match(rest)
    if not m:
        raise NotImplementedError(f"{block}: LoRA target {rest!r} is not a linear layer of the transformer blocks")
    if m.group(2) is None:
        return f"{block}.{rest}", False
    t, leaf = m.group(2), m.group(3)
    if leaf.startswith("attn"):
        attn, proj = leaf[:5], leaf[6:]
        return f"{block}.transformer_blocks.{t}.{attn}.processor.{'to_out' if proj == 'to_out_0' else proj}_lora", True
    return f"{block}.transformer_blocks.{t}.{'ff.net.0.proj' if leaf == 'ff_net_0_proj' else 'ff.net.2'}", False


def convert_kohya_lora_to_diffusers(state_dict: Mapping[str, torch.Tensor], layers_per_block: int = 2):
    """-> (unet_state_dict, network_alphas, passthrough).  unet_state_dict keys: `unet.<path>.lora.down.weight` /
    `unet.<attn>.processor.to_q_lora.down.weight` (+ `.up.`); network_alphas: {`unet.<...>.alpha`: float} named as the
    reference names them (for attention projections the alpha hangs off the full down key)."""
    unet_sd: Dict[str, torch.Tensor] = {}
    alphas: Dict[str, float] = {}
    passthrough: Dict[str, torch.Tensor] = {}
    seen = {}
    for key, val in state_dict.items():
        if not key.startswith("lora_unet_"):
            passthrough[key] = val
            continue
        for suf in _SUFFIXES:
            if key.endswith(suf):
                name, which = key[len("lora_unet_"):-len(suf)], suf
                break
        else:
            raise ValueError(f"{key}: expected a .lora_down.weight, .lora_up.weight or .alpha entry")
        block, rest = _block_address(name, layers_per_block)
        path, is_attn = _module_path(block, rest)
        stem = f"unet.{path}" if is_attn else f"unet.{path}.lora"
        if which == ".alpha":
            a = float(val.item() if isinstance(val, torch.Tensor) else val)
            alphas[(stem + ".down.weight.alpha") if is_attn else f"unet.{path}.alpha"] = a
        else:
            unet_sd[stem + (".down.weight" if which == ".lora_down.weight" else ".up.weight")] = val
            seen.setdefault(stem, set()).add(which)
    for stem, parts in seen.items():
        if parts != {".lora_down.weight", ".lora_up.weight"}:
            raise ValueError(f"{stem}: needs both lora_down and lora_up")
    return unet_sd, alphas, passthrough
