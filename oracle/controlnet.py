"""CPU fp32 restatement of ControlNetModel.forward for the SDXL configuration (checker, not product).

Follows diffusers-hf/src/diffusers/models/controlnet.py: conditioning embedding :84-126, constructor :201-466
(SDXL arguments: the UNet's encoder, conditioning_embedding_out_channels (16, 32, 96, 256), zero-initialised
1x1 `controlnet_down_blocks` / `controlnet_mid_block` :384-430), forward :687-847 (Katz's default
conditioning_scale = 0.5, :693).  The encoder blocks are the ones pinned by the reference's known-answer tests
(oracle/blocks.py).  Pinned here (tests/test_oracle_controlnet.py): freshly constructed (zero-initialised zero
convs, :58-61 zero_module) every residual is exactly zero; with identity zero convs and a zero conditioning
embedding the residuals equal conditioning_scale x the UNet encoder's skips (from_unet semantics, :432-506);
residual shapes equal unet_2d_condition.py:539-563; and numerically against outputs of the reference's own
ControlNetModel (from_unet, random non-zero zero convolutions and conditioning embedding, conditioning_scale 0.5 and
1.0) on a tiny SDXL-topology configuration, <= 1e-4 relative (tests/golden/unet_tiny_reference.safetensors).
"""
from __future__ import annotations

from typing import Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import blocks as Bk
from .unet_sdxl import UNetConfig


def zero_module(m: nn.Module) -> nn.Module:
    for p in m.parameters():
        nn.init.zeros_(p)
    return m


class ControlNetConditioningEmbedding(nn.Module):
    def __init__(self, conditioning_embedding_channels: int, conditioning_channels: int = 3,
                 block_out_channels: Tuple[int, ...] = (16, 32, 96, 256)):
        super().__init__()
        self.conv_in = nn.Conv2d(conditioning_channels, block_out_channels[0], 3, padding=1)
        self.blocks = nn.ModuleList()
        for i in range(len(block_out_channels) - 1):
            cin, cout = block_out_channels[i], block_out_channels[i + 1]
            self.blocks.append(nn.Conv2d(cin, cin, 3, padding=1))
            self.blocks.append(nn.Conv2d(cin, cout, 3, padding=1, stride=2))
        self.conv_out = zero_module(nn.Conv2d(block_out_channels[-1], conditioning_embedding_channels, 3, padding=1))

    def forward(self, conditioning):
        e = F.silu(self.conv_in(conditioning))
        for b in self.blocks:
            e = F.silu(b(e))
        return self.conv_out(e)


class ControlNetModel(nn.Module):
    def __init__(self, cfg: UNetConfig, conditioning_embedding_out_channels: Tuple[int, ...] = (16, 32, 96, 256)):
        super().__init__()
        self.cfg = cfg
        boc = cfg.block_out_channels
        ted = boc[0] * 4
        self.conv_in = nn.Conv2d(cfg.in_channels, boc[0], 3, padding=1)
        self.time_embedding = Bk.TimestepEmbedding(boc[0], ted)
        self.add_embedding = Bk.TimestepEmbedding(cfg.projection_class_embeddings_input_dim, ted)
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
                self.down_blocks.append(Bk.DownBlock2D(**common))
            else:
                self.down_blocks.append(Bk.CrossAttnDownBlock2D(
                    **common, transformer_layers_per_block=cfg.transformer_layers_per_block[i],
                    num_attention_heads=cfg.num_attention_heads[i], cross_attention_dim=cfg.cross_attention_dim,
                    use_linear_projection=cfg.use_linear_projection))
            for _ in range(cfg.layers_per_block + (0 if final else 1)):
                self.controlnet_down_blocks.append(zero_module(nn.Conv2d(out_ch, out_ch, 1)))
        self.controlnet_mid_block = zero_module(nn.Conv2d(boc[-1], boc[-1], 1))
        self.mid_block = Bk.UNetMidBlock2DCrossAttn(
            in_channels=boc[-1], temb_channels=ted, transformer_layers_per_block=cfg.transformer_layers_per_block[-1],
            resnet_eps=cfg.norm_eps, resnet_groups=cfg.norm_num_groups, num_attention_heads=cfg.num_attention_heads[-1],
            cross_attention_dim=cfg.cross_attention_dim, use_linear_projection=cfg.use_linear_projection)

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

    def forward(self, sample, timestep, encoder_hidden_states, controlnet_cond, conditioning_scale: float = 0.5,
                added_cond_kwargs=None):
        emb = self.embed(sample, timestep, added_cond_kwargs)
        sample = self.conv_in(sample)
        sample = sample + self.controlnet_cond_embedding(controlnet_cond)
        skips = (sample,)
        for blk in self.down_blocks:
            sample, res = blk(sample, emb, encoder_hidden_states)
            skips += res
        sample = self.mid_block(sample, emb, encoder_hidden_states)
        down = [zc(s) * conditioning_scale for s, zc in zip(skips, self.controlnet_down_blocks)]
        mid = self.controlnet_mid_block(sample) * conditioning_scale
        return down, mid
