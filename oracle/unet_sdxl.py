"""CPU fp32 restatement of UNet2DConditionModel.forward for the SDXL configuration (checker, not product).

Follows diffusers-hf/src/diffusers/models/unets/unet_2d_condition.py: constructor :279-507 (SDXL
arguments), time / text_time embeddings :997-1021, :1055-1075, down + mid :1127-1252, ControlNet
residual injection + up + post-process :1254-1341.  The blocks it wires are pinned by the reference's
known-answer tests (oracle/blocks.py); the wiring itself is pinned numerically by outputs of the
reference's own UNet2DConditionModel on a tiny SDXL-topology configuration (depths 1 / 2 / 3, text_time
conditioning, with and without the 9 + 1 residuals; tests/golden/unet_tiny_reference.safetensors, <= 1e-4) and
structurally: the LoRA-able linear names equal the 722 keys of the reference's
lora_info_shm/*_key_match_unet.json fixture and the skip tensors have the shapes of
unet_2d_condition.py:539-563 (tests/test_oracle_unet.py).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import blocks as Bk
from . import ops as O


@dataclass
class UNetConfig:
    in_channels: int = 4
    out_channels: int = 4
    block_out_channels: Tuple[int, ...] = (320, 640, 1280)
    down_block_types: Tuple[str, ...] = ("DownBlock2D", "CrossAttnDownBlock2D", "CrossAttnDownBlock2D")
    up_block_types: Tuple[str, ...] = ("CrossAttnUpBlock2D", "CrossAttnUpBlock2D", "UpBlock2D")
    layers_per_block: int = 2
    transformer_layers_per_block: Tuple[int, ...] = (1, 2, 10)
    num_attention_heads: Tuple[int, ...] = (5, 10, 20)   # SDXL stores these under `attention_head_dim`
    cross_attention_dim: int = 2048
    norm_num_groups: int = 32
    norm_eps: float = 1e-5
    addition_time_embed_dim: int = 256
    projection_class_embeddings_input_dim: int = 2816
    use_linear_projection: bool = True

    @staticmethod
    def sdxl() -> "UNetConfig":
        return UNetConfig()

    @staticmethod
    def tiny() -> "UNetConfig":
        """Same topology, head_dim 64, small widths: for parity tests that must run in seconds."""
        return UNetConfig(block_out_channels=(64, 128, 256), transformer_layers_per_block=(1, 1, 2),
                          num_attention_heads=(1, 2, 4), cross_attention_dim=128, addition_time_embed_dim=32,
                          projection_class_embeddings_input_dim=64 + 6 * 32)


class UNet2DConditionModel(nn.Module):
    def __init__(self, cfg: UNetConfig):
        super().__init__()
        self.cfg = cfg
        boc = cfg.block_out_channels
        ted = boc[0] * 4
        self.conv_in = nn.Conv2d(cfg.in_channels, boc[0], 3, padding=1)
        self.time_embedding = Bk.TimestepEmbedding(boc[0], ted)
        self.add_embedding = Bk.TimestepEmbedding(cfg.projection_class_embeddings_input_dim, ted)
        n = len(boc)
        self.down_blocks = nn.ModuleList()
        out_ch = boc[0]
        for i, typ in enumerate(cfg.down_block_types):
            in_ch, out_ch = out_ch, boc[i]
            final = i == n - 1
            common = dict(in_channels=in_ch, out_channels=out_ch, temb_channels=ted, num_layers=cfg.layers_per_block,
                          resnet_eps=cfg.norm_eps, resnet_groups=cfg.norm_num_groups, add_downsample=not final)
            if typ == "DownBlock2D":
                self.down_blocks.append(Bk.DownBlock2D(**common))
            else:
                self.down_blocks.append(Bk.CrossAttnDownBlock2D(
                    **common, transformer_layers_per_block=cfg.transformer_layers_per_block[i],
                    num_attention_heads=cfg.num_attention_heads[i], cross_attention_dim=cfg.cross_attention_dim,
                    use_linear_projection=cfg.use_linear_projection))
        self.mid_block = Bk.UNetMidBlock2DCrossAttn(
            in_channels=boc[-1], temb_channels=ted, transformer_layers_per_block=cfg.transformer_layers_per_block[-1],
            resnet_eps=cfg.norm_eps, resnet_groups=cfg.norm_num_groups, num_attention_heads=cfg.num_attention_heads[-1],
            cross_attention_dim=cfg.cross_attention_dim, use_linear_projection=cfg.use_linear_projection)
        self.up_blocks = nn.ModuleList()
        rev = list(reversed(boc))
        rev_heads = list(reversed(cfg.num_attention_heads))
        rev_tl = list(reversed(cfg.transformer_layers_per_block))
        out_ch = rev[0]
        for i, typ in enumerate(cfg.up_block_types):
            prev, out_ch = out_ch, rev[i]
            in_ch = rev[min(i + 1, n - 1)]
            final = i == n - 1
            common = dict(in_channels=in_ch, out_channels=out_ch, prev_output_channel=prev, temb_channels=ted,
                          num_layers=cfg.layers_per_block + 1, resnet_eps=cfg.norm_eps,
                          resnet_groups=cfg.norm_num_groups, add_upsample=not final)
            if typ == "UpBlock2D":
                self.up_blocks.append(Bk.UpBlock2D(**common))
            else:
                self.up_blocks.append(Bk.CrossAttnUpBlock2D(
                    **common, transformer_layers_per_block=rev_tl[i], num_attention_heads=rev_heads[i],
                    cross_attention_dim=cfg.cross_attention_dim, use_linear_projection=cfg.use_linear_projection))
        self.conv_norm_silu = nn.Sequential(*Bk.fused_norm_silu(boc[0], cfg.norm_num_groups, cfg.norm_eps))
        self.conv_out = nn.Conv2d(boc[0], cfg.out_channels, 3, padding=1)

    # ---- LoRA bookkeeping --------------------------------------------------------------------
    def lora_linears(self) -> Dict[str, Bk.OracleLoRALinear]:
        return {n: m for n, m in self.named_modules() if isinstance(m, Bk.OracleLoRALinear)}

    def add_adapter(self, name: str, tensors: Dict[str, Tuple[torch.Tensor, torch.Tensor]], alpha=None, weight=1.0):
        """tensors: {linear module name: (down [r,in], up [out,r])}."""
        lin = self.lora_linears()
        for k, (down, up) in tensors.items():
            lin[k].add_adapter(name, down, up, alpha, weight)

    def set_adapters(self, names: Sequence[str], weights: Optional[Sequence[float]] = None):
        weights = [1.0] * len(names) if weights is None else list(weights)
        for m in self.lora_linears().values():
            m.active = [n for n in names if n in m.adapters]
            for n, w in zip(names, weights):
                if n in m.adapters:
                    m.adapters[n]["weight"] = w

    # ---- forward ------------------------------------------------------------------------------
    def embed(self, sample, timestep, added_cond_kwargs):
        cfg = self.cfg
        B = sample.shape[0]
        t = timestep if torch.is_tensor(timestep) else torch.tensor([timestep], dtype=torch.float32)
        t = t.reshape(-1).expand(B) if t.numel() == 1 else t
        t_emb = Bk.get_timestep_embedding(t, cfg.block_out_channels[0], flip_sin_to_cos=True, downscale_freq_shift=0)
        emb = self.time_embedding(t_emb.to(sample.dtype))
        text_embeds, time_ids = added_cond_kwargs["text_embeds"], added_cond_kwargs["time_ids"]
        tid = Bk.get_timestep_embedding(time_ids.flatten(), cfg.addition_time_embed_dim, flip_sin_to_cos=True,
                                        downscale_freq_shift=0).reshape(B, -1)
        add = torch.cat([text_embeds, tid.to(text_embeds.dtype)], dim=-1)
        return emb + self.add_embedding(add.to(sample.dtype))

    def forward(self, sample, timestep, encoder_hidden_states, added_cond_kwargs,
                down_block_additional_residuals=None, mid_block_additional_residual=None, return_skips=False):
        emb = self.embed(sample, timestep, added_cond_kwargs)
        sample = self.conv_in(sample)
        skips = (sample,)
        for blk in self.down_blocks:
            sample, res = blk(sample, emb, encoder_hidden_states)
            skips += res
        sample = self.mid_block(sample, emb, encoder_hidden_states)
        if return_skips:
            return skips, sample
        if down_block_additional_residuals is not None:
            skips = tuple(O.residual_add(s, [r]) for s, r in zip(skips, down_block_additional_residuals))
        if mid_block_additional_residual is not None:
            sample = O.residual_add(sample, [mid_block_additional_residual])
        for blk in self.up_blocks:
            n = len(blk.resnets)
            res, skips = skips[-n:], skips[:-n]
            sample = blk(sample, res, emb, encoder_hidden_states)
        sample = self.conv_norm_silu(sample)
        return self.conv_out(sample)
