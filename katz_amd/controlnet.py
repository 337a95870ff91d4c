"""ControlNetModel (SDXL configuration) on the katz_hip kernels.

Drop-in for the reference's model at the call boundary
(diffusers-hf/src/diffusers/models/controlnet.py: constructor :201-466, forward :687-847, conditioning
embedding :84-126): same forward arguments, Katz's default `conditioning_scale = 0.5` (:693), same module /
state-dict names.  It is the UNet's encoder (the same `DownBlock2D` / `CrossAttnDownBlock2D` /
`UNetMidBlock2DCrossAttn` modules and kernels), a small convolutional embedding of the conditioning image
added after `conv_in` (:780-783), and one 1x1 "zero convolution" per skip tensor (:818-824), whose outputs,
times `conditioning_scale`, are the residuals `UNet2DConditionModel.forward` takes as
`down_block_additional_residuals` / `mid_block_additional_residual`.
"""
from __future__ import annotations

from typing import Any, Dict, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops
from .layers import Conv3x3, TimestepEmbedding
from .unet_2d_condition import UNet2DConditionModel, UNetConfig
from .unet_blocks import CrossAttnDownBlock2D, DownBlock2D, UNetMidBlock2DCrossAttn


def zero_module(m: nn.Module) -> nn.Module:
    for p in m.parameters():
        nn.init.zeros_(p)
    return m


def conv1x1_scaled(x: torch.Tensor, conv: nn.Conv2d, scale: float, cache: Optional[dict] = None) -> torch.Tensor:
    """(1x1 convolution of a channels_last tensor) * scale: a linear layer over the channels of every pixel, with the
    scale folded into the layer, scale * (W x + b) = (scale W) x + scale b, so the residual leaves the GEMM epilogue
    finished (controlnet.py:818-824 followed by the `sample * conditioning_scale` of :833-835).  Exact for powers of
    two (Katz's default 0.5, upstream's 1.0); otherwise the scaled weights are rounded to bf16 once instead of the
    output twice.  cache: {id(conv): (key, weight, bias)} kept by the caller, rebuilt when scale or weights change."""
    nb, c, hh, ww = x.shape
    x = x.contiguous(memory_format=torch.channels_last)
    w, b = conv.weight.reshape(conv.out_channels, c), conv.bias
    if scale != 1.0:
        key = (float(scale), conv.weight._version, conv.weight.data_ptr(), None if b is None else b._version)
        hit = None if cache is None else cache.get(id(conv))
        if hit is None or hit[0] != key:
            with torch.no_grad():
                hit = (key, (w.float() * scale).to(w.dtype).contiguous(),
                       None if b is None else (b.float() * scale).to(b.dtype))
            if cache is not None and not (x.is_cuda and torch.cuda.is_current_stream_capturing()):
                cache[id(conv)] = hit     # tensors made during a capture belong to that graph: do not keep them
        w, b = hit[1], hit[2]
    y = ops.lora_linear(x.permute(0, 2, 3, 1).reshape(nb * hh * ww, c), w, b)
    return y.view(nb, hh, ww, conv.out_channels).permute(0, 3, 1, 2)


class ControlNetConditioningEmbedding(nn.Module):
    """controlnet.py:84-126: conv_in, (conv, stride-2 conv) x 3 with SiLU after each, zero-initialised conv_out."""

    def __init__(self, conditioning_embedding_channels: int, conditioning_channels: int = 3,
                 block_out_channels: Tuple[int, ...] = (16, 32, 96, 256)):
        super().__init__()
        self.conv_in = Conv3x3(conditioning_channels, block_out_channels[0])
        self.blocks = nn.ModuleList()
        for i in range(len(block_out_channels) - 1):
            cin, cout = block_out_channels[i], block_out_channels[i + 1]
            self.blocks.append(Conv3x3(cin, cin))
            self.blocks.append(Conv3x3(cin, cout, stride=2))
        self.conv_out = zero_module(Conv3x3(block_out_channels[-1], conditioning_embedding_channels))

    def forward(self, conditioning):
        e = F.silu(self.conv_in(conditioning))
        for b in self.blocks:
            e = F.silu(b(e))
        return self.conv_out(e)


class ControlNetModel(nn.Module):
    def __init__(self, cfg: Optional[UNetConfig] = None, conditioning_embedding_out_channels: Tuple[int, ...] = (16, 32, 96, 256)):
        super().__init__()
        cfg = cfg or UNetConfig.sdxl()
        self.cfg = cfg
        boc = cfg.block_out_channels
        ted = boc[0] * 4
        self.conv_in = Conv3x3(cfg.in_channels, boc[0])
        self.time_embedding = TimestepEmbedding(boc[0], ted)
        self.add_embedding = TimestepEmbedding(cfg.projection_class_embeddings_input_dim, ted)
        self.controlnet_cond_embedding = ControlNetConditioningEmbedding(boc[0], 3, conditioning_embedding_out_channels)
        self.down_blocks = nn.ModuleList()
        self.controlnet_down_blocks = nn.ModuleList()
        out_ch = boc[0]
        self.controlnet_down_blocks.append(zero_module(nn.Conv2d(out_ch, out_ch, 1)))
        n = len(boc)
        for i, typ in enumerate(cfg.down_block_types):
            in_ch, out_ch = out_ch, boc[i]
            final = i == n - 1
            common = dict(in_channels=in_ch, out_channels=out_ch, temb_channels=ted, num_layers=cfg.layers_per_block,
                          resnet_eps=cfg.norm_eps, resnet_groups=cfg.norm_num_groups, add_downsample=not final)
            if typ == "DownBlock2D":
                self.down_blocks.append(DownBlock2D(**common))
            elif typ == "CrossAttnDownBlock2D":
                self.down_blocks.append(CrossAttnDownBlock2D(
                    **common, transformer_layers_per_block=cfg.transformer_layers_per_block[i],
                    num_attention_heads=cfg.num_attention_heads[i], cross_attention_dim=cfg.cross_attention_dim,
                    use_linear_projection=cfg.use_linear_projection))
            else:
                raise ValueError(f"unsupported down block {typ}")
            for _ in range(cfg.layers_per_block + (0 if final else 1)):
                self.controlnet_down_blocks.append(zero_module(nn.Conv2d(out_ch, out_ch, 1)))
        self.controlnet_mid_block = zero_module(nn.Conv2d(boc[-1], boc[-1], 1))
        self.mid_block = UNetMidBlock2DCrossAttn(
            in_channels=boc[-1], temb_channels=ted, transformer_layers_per_block=cfg.transformer_layers_per_block[-1],
            resnet_eps=cfg.norm_eps, resnet_groups=cfg.norm_num_groups, num_attention_heads=cfg.num_attention_heads[-1],
            cross_attention_dim=cfg.cross_attention_dim, use_linear_projection=cfg.use_linear_projection)
        self._ctx_kv = None
        self._zero_conv_cache: Dict[int, tuple] = {}
        self._register_load_state_dict_pre_hook(UNet2DConditionModel._remap_upstream_keys)

    @classmethod
    def from_unet(cls, unet: UNet2DConditionModel, conditioning_embedding_out_channels=(16, 32, 96, 256),
                  load_weights_from_unet: bool = True) -> "ControlNetModel":
        """controlnet.py:432-506: a ControlNet whose encoder starts as a copy of the UNet's."""
        cn = cls(unet.cfg, conditioning_embedding_out_channels)
        if load_weights_from_unet:
            for name in ("conv_in", "time_embedding", "add_embedding", "down_blocks", "mid_block"):
                getattr(cn, name).load_state_dict(getattr(unet, name).state_dict())
        return cn

    def to_runtime(self, device="cuda", dtype=torch.bfloat16) -> "ControlNetModel":
        self.to(device=device, dtype=dtype)
        self.to(memory_format=torch.channels_last)
        self.prepare()
        return self.eval()

    def embed_condition(self, controlnet_cond: torch.Tensor) -> torch.Tensor:
        """controlnet_cond_embedding(image) (:84-126, applied at :780), channels_last bf16."""
        cond = controlnet_cond.to(torch.bfloat16).contiguous(memory_format=torch.channels_last)
        return self.controlnet_cond_embedding(cond).contiguous(memory_format=torch.channels_last)

    prepare = UNet2DConditionModel.prepare
    lora_linears = UNet2DConditionModel.lora_linears
    _embed = UNet2DConditionModel._embed

    def forward(self, sample, timestep, encoder_hidden_states, controlnet_cond, conditioning_scale: float = 0.5,
                class_labels=None, timestep_cond=None, attention_mask=None,
                added_cond_kwargs: Optional[Dict[str, torch.Tensor]] = None,
                cross_attention_kwargs: Optional[Dict[str, Any]] = None, guess_mode: bool = False,
                return_dict: bool = False, cond_embedding: Optional[torch.Tensor] = None):
        """controlnet.py:687-847.  cond_embedding (not in the reference): the result of embed_condition(controlnet_cond)
        computed earlier -- in a denoise loop the image, and so its embedding, is the same in every step."""
        for name, val in (("class_labels", class_labels), ("timestep_cond", timestep_cond), ("attention_mask", attention_mask)):
            if val is not None:
                raise NotImplementedError(f"`{name}` is not used on the SDXL ControlNet path and is not implemented")
        if guess_mode:
            raise NotImplementedError("guess_mode (logspace residual scales, controlnet.py:827-831) is not implemented")
        if sample.dtype != torch.bfloat16 or not sample.is_contiguous(memory_format=torch.channels_last):
            sample = sample.to(torch.bfloat16).contiguous(memory_format=torch.channels_last)
        ctx = encoder_hidden_states.to(torch.bfloat16).contiguous()
        if sample.is_cuda:
            ops.split_counters_reset(sample.device)   # one fill per step clears the in-launch shrinks' counters
        with ops.weight_prefetch_scope(self):   # hints are learned from, and point into, this model's own last pass
            if self._ctx_kv is None:
                self.prepare()
            if not getattr(self, "context_kv_ready", False):   # (a denoise loop projects its one text context once, not per step)
                self._ctx_kv.run(ctx)
            emb = self._embed(sample, timestep, added_cond_kwargs)
            temb_act = F.silu(emb)
            self._temb_proj.run(temb_act)   # time_emb_proj of all resnets, batched per width
            if cond_embedding is None:
                cond_embedding = self.embed_condition(controlnet_cond)
            # conv_in(sample) + embedding (:780-783): the add runs in the convolution's epilogue
            sample = self.conv_in(sample, residual=cond_embedding)
            skips = (sample,)
            for blk in self.down_blocks:
                sample, res = blk(sample, temb_act, ctx)
                skips += res
            sample = self.mid_block(sample, temb_act, ctx)
            zc_cache = self._zero_conv_cache
            down = [conv1x1_scaled(s, zc, conditioning_scale, zc_cache) for s, zc in zip(skips, self.controlnet_down_blocks)]
            mid = conv1x1_scaled(sample, self.controlnet_mid_block, conditioning_scale, zc_cache)
        if not return_dict:
            return (down, mid)
        return {"down_block_res_samples": down, "mid_block_res_sample": mid}
