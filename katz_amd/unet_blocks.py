"""Down / mid / up blocks of the SDXL UNet on the katz_hip layers
(diffusers-hf/src/diffusers/models/unets/unet_2d_blocks.py: DownBlock2D :1303-1392, CrossAttnDownBlock2D
:1140-1300, UNetMidBlock2DCrossAttn :744-890, CrossAttnUpBlock2D :2382-2555, UpBlock2D :2558-2670).

`temb_act` is silu(temb), shared by every resnet of the step.  The up blocks take, per skip tensor, the
list of ControlNet residual tensors to add to it (possibly empty): the add is folded into the
channel concat that feeds the resnet (one kernel instead of add + cat).
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch
import torch.nn as nn

from . import ops
from .layers import Downsample2D, ResnetBlock2D, Transformer2DModel, Upsample2D


def _as_list(v, n):
    return [v] * n if isinstance(v, int) else list(v)


class DownBlock2D(nn.Module):
    has_cross_attention = False

    def __init__(self, in_channels, out_channels, temb_channels, num_layers=1, resnet_eps=1e-6, resnet_groups=32,
                 add_downsample=True, downsample_padding=1):
        super().__init__()
        self.resnets = nn.ModuleList([
            ResnetBlock2D(in_channels=in_channels if i == 0 else out_channels, out_channels=out_channels,
                          temb_channels=temb_channels, eps=resnet_eps, groups=resnet_groups)
            for i in range(num_layers)])
        self.downsamplers = nn.ModuleList([Downsample2D(out_channels, True, out_channels, downsample_padding, "op",
                                                        stats_groups=resnet_groups)]) \
            if add_downsample else None

    def forward(self, hidden_states, temb_act, encoder_hidden_states=None):
        outs = ()
        for resnet in self.resnets:
            hidden_states = resnet(hidden_states, temb_act)
            outs += (hidden_states,)
        if self.downsamplers is not None:
            hidden_states = self.downsamplers[0](hidden_states)
            outs += (hidden_states,)
        return hidden_states, outs


class CrossAttnDownBlock2D(nn.Module):
    has_cross_attention = True

    def __init__(self, in_channels, out_channels, temb_channels, num_layers=1, transformer_layers_per_block=1,
                 resnet_eps=1e-6, resnet_groups=32, num_attention_heads=1, cross_attention_dim=1280,
                 add_downsample=True, downsample_padding=1, use_linear_projection=True):
        super().__init__()
        tl = _as_list(transformer_layers_per_block, num_layers)
        resnets, attns = [], []
        for i in range(num_layers):
            resnets.append(ResnetBlock2D(in_channels=in_channels if i == 0 else out_channels, out_channels=out_channels,
                                         temb_channels=temb_channels, eps=resnet_eps, groups=resnet_groups))
            attns.append(Transformer2DModel(num_attention_heads, out_channels // num_attention_heads, out_channels,
                                            num_layers=tl[i], cross_attention_dim=cross_attention_dim,
                                            norm_num_groups=resnet_groups, use_linear_projection=use_linear_projection))
        self.attentions = nn.ModuleList(attns)
        self.resnets = nn.ModuleList(resnets)
        self.downsamplers = nn.ModuleList([Downsample2D(out_channels, True, out_channels, downsample_padding, "op",
                                                        stats_groups=resnet_groups)]) \
            if add_downsample else None

    def forward(self, hidden_states, temb_act, encoder_hidden_states=None):
        outs = ()
        for resnet, attn in zip(self.resnets, self.attentions):
            hidden_states = resnet(hidden_states, temb_act)
            hidden_states = attn(hidden_states, encoder_hidden_states)
            outs += (hidden_states,)
        if self.downsamplers is not None:
            hidden_states = self.downsamplers[0](hidden_states)
            outs += (hidden_states,)
        return hidden_states, outs


class UNetMidBlock2DCrossAttn(nn.Module):
    has_cross_attention = True

    def __init__(self, in_channels, temb_channels, num_layers=1, transformer_layers_per_block=1, resnet_eps=1e-6,
                 resnet_groups=32, num_attention_heads=1, cross_attention_dim=1280, use_linear_projection=True):
        super().__init__()
        tl = _as_list(transformer_layers_per_block, num_layers)
        mk = lambda: ResnetBlock2D(in_channels=in_channels, out_channels=in_channels, temb_channels=temb_channels,
                                   eps=resnet_eps, groups=resnet_groups)
        resnets, attns = [mk()], []
        for i in range(num_layers):
            attns.append(Transformer2DModel(num_attention_heads, in_channels // num_attention_heads, in_channels,
                                            num_layers=tl[i], cross_attention_dim=cross_attention_dim,
                                            norm_num_groups=resnet_groups, use_linear_projection=use_linear_projection))
            resnets.append(mk())
        self.attentions = nn.ModuleList(attns)
        self.resnets = nn.ModuleList(resnets)

    def forward(self, hidden_states, temb_act, encoder_hidden_states=None):
        hidden_states = self.resnets[0](hidden_states, temb_act)
        for attn, resnet in zip(self.attentions, self.resnets[1:]):
            hidden_states = attn(hidden_states, encoder_hidden_states)
            hidden_states = resnet(hidden_states, temb_act)
        return hidden_states


def _up_resnets(in_channels, prev_output_channel, out_channels, temb_channels, num_layers, resnet_eps, resnet_groups):
    resnets = []
    for i in range(num_layers):
        res_skip = in_channels if (i == num_layers - 1) else out_channels
        res_in = prev_output_channel if i == 0 else out_channels
        resnets.append(ResnetBlock2D(in_channels=res_in + res_skip, out_channels=out_channels,
                                     temb_channels=temb_channels, eps=resnet_eps, groups=resnet_groups))
    return resnets


class UpBlock2D(nn.Module):
    has_cross_attention = False

    def __init__(self, in_channels, prev_output_channel, out_channels, temb_channels, num_layers=1, resnet_eps=1e-6,
                 resnet_groups=32, add_upsample=True):
        super().__init__()
        self.resnets = nn.ModuleList(_up_resnets(in_channels, prev_output_channel, out_channels, temb_channels,
                                                 num_layers, resnet_eps, resnet_groups))
        self.upsamplers = nn.ModuleList([Upsample2D(out_channels, True, out_channels)]) if add_upsample else None

    def forward(self, hidden_states, res_hidden_states_tuple, res_additional, temb_act, encoder_hidden_states=None,
                upsample_size=None):
        for resnet in self.resnets:
            skip, extra = res_hidden_states_tuple[-1], res_additional[-1]
            res_hidden_states_tuple, res_additional = res_hidden_states_tuple[:-1], res_additional[:-1]
            hidden_states = ops.concat_residual(hidden_states, skip, extra)
            hidden_states = resnet(hidden_states, temb_act)
        if self.upsamplers is not None:
            hidden_states = self.upsamplers[0](hidden_states, upsample_size)
        return hidden_states


class CrossAttnUpBlock2D(nn.Module):
    has_cross_attention = True

    def __init__(self, in_channels, out_channels, prev_output_channel, temb_channels, num_layers=1,
                 transformer_layers_per_block=1, resnet_eps=1e-6, resnet_groups=32, num_attention_heads=1,
                 cross_attention_dim=1280, add_upsample=True, use_linear_projection=True):
        super().__init__()
        tl = _as_list(transformer_layers_per_block, num_layers)
        self.resnets = nn.ModuleList(_up_resnets(in_channels, prev_output_channel, out_channels, temb_channels,
                                                 num_layers, resnet_eps, resnet_groups))
        self.attentions = nn.ModuleList([
            Transformer2DModel(num_attention_heads, out_channels // num_attention_heads, out_channels, num_layers=tl[i],
                               cross_attention_dim=cross_attention_dim, norm_num_groups=resnet_groups,
                               use_linear_projection=use_linear_projection) for i in range(num_layers)])
        self.upsamplers = nn.ModuleList([Upsample2D(out_channels, True, out_channels)]) if add_upsample else None

    def forward(self, hidden_states, res_hidden_states_tuple, res_additional, temb_act, encoder_hidden_states=None,
                upsample_size=None):
        for resnet, attn in zip(self.resnets, self.attentions):
            skip, extra = res_hidden_states_tuple[-1], res_additional[-1]
            res_hidden_states_tuple, res_additional = res_hidden_states_tuple[:-1], res_additional[:-1]
            hidden_states = ops.concat_residual(hidden_states, skip, extra)
            hidden_states = resnet(hidden_states, temb_act)
            hidden_states = attn(hidden_states, encoder_hidden_states)
        if self.upsamplers is not None:
            hidden_states = self.upsamplers[0](hidden_states, upsample_size)
        return hidden_states
