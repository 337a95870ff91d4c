"""CPU fp32 restatement of the reference's SDXL UNet building blocks (checker, not product).

Modules are built in the reference's construction order with torch's default initialisation, so the
reference's seeded known-answer tests (diffusers-hf/tests/models/test_layers_utils.py,
diffusers-hf/tests/models/unets/test_unet_2d_blocks.py) reproduce -- that is what pins this file
(tests/test_oracle_kats.py).  Module / parameter names are the reference's (Katz fork: norm_silu1.0,
norm_silu2.0, conv_norm_silu.0), so state dicts are interchangeable with the product modules.

Every LoRA-able nn.Linear is an `OracleLoRALinear`, which evaluates oracle.ops.lora_linear over its
active adapters.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops as O


# ----------------------------------------------------------------------------------- embeddings
def get_timestep_embedding(timesteps, embedding_dim: int, flip_sin_to_cos: bool = False,
                           downscale_freq_shift: float = 1, scale: float = 1, max_period: int = 10000):
    """Sinusoidal embedding, diffusers-hf/src/diffusers/models/embeddings.py:26-66."""
    half = embedding_dim // 2
    exponent = -math.log(max_period) * torch.arange(0, half, dtype=torch.float32, device=timesteps.device)
    exponent = exponent / (half - downscale_freq_shift)
    emb = timesteps[:, None].float() * torch.exp(exponent)[None, :]
    emb = scale * emb
    emb = torch.cat([torch.sin(emb), torch.cos(emb)], dim=-1)
    if flip_sin_to_cos:
        emb = torch.cat([emb[:, half:], emb[:, :half]], dim=-1)
    if embedding_dim % 2 == 1:
        emb = F.pad(emb, (0, 1, 0, 0))
    return emb


class TimestepEmbedding(nn.Module):
    """linear_1 -> SiLU -> linear_2, diffusers-hf/src/diffusers/models/embeddings.py:190-235."""

    def __init__(self, in_channels: int, time_embed_dim: int):
        super().__init__()
        self.linear_1 = nn.Linear(in_channels, time_embed_dim)
        self.linear_2 = nn.Linear(time_embed_dim, time_embed_dim)

    def forward(self, sample):
        return self.linear_2(F.silu(self.linear_1(sample)))


# ----------------------------------------------------------------------------------- LoRA linear
class OracleLoRALinear(nn.Linear):
    """nn.Linear plus named adapters; forward = oracle.ops.lora_linear over the active ones.
    Adapter bookkeeping mirrors peft's per-layer state as driven by
    diffusers-hf/src/diffusers/utils/peft_utils.py:238-269."""

    def __init__(self, in_features, out_features, bias=True):
        super().__init__(in_features, out_features, bias=bias)
        self.adapters: Dict[str, dict] = {}
        self.active: List[str] = []
        self.global_scale = 1.0

    def add_adapter(self, name, down, up, alpha=None, weight=1.0):
        self.adapters[name] = dict(down=down, up=up, alpha=alpha, weight=weight)

    def multiplier(self, name):
        a = self.adapters[name]
        r = a["down"].shape[0]
        alpha = r if a["alpha"] is None else a["alpha"]
        return a["weight"] * alpha / r * self.global_scale

    def forward(self, x, residual=None):
        ads = [(self.adapters[n]["down"], self.adapters[n]["up"], self.multiplier(n)) for n in self.active]
        return O.lora_linear(x, self.weight, self.bias, ads, residual)


# ----------------------------------------------------------------------------------- norm helpers
def fused_norm_silu(num_channels, norm_num_groups, eps, affine=True):
    """[GroupNorm, SiLU] (env flag off), diffusers-hf/src/diffusers/models/normalization.py:30-37."""
    return [nn.GroupNorm(norm_num_groups, num_channels, eps=eps, affine=affine), nn.SiLU()]


class Downsample2D(nn.Module):
    """diffusers-hf/src/diffusers/models/downsampling.py:69-149."""

    def __init__(self, channels, use_conv=False, out_channels=None, padding=1, name="conv"):
        super().__init__()
        self.channels, self.out_channels = channels, out_channels or channels
        self.use_conv, self.padding = use_conv, padding
        if use_conv:
            self.conv = nn.Conv2d(channels, self.out_channels, 3, stride=2, padding=padding)
        else:
            assert self.channels == self.out_channels
            self.conv = nn.AvgPool2d(kernel_size=2, stride=2)

    def forward(self, x):
        if self.use_conv and self.padding == 0:
            x = F.pad(x, (0, 1, 0, 1), mode="constant", value=0)
        return self.conv(x)


class Upsample2D(nn.Module):
    """diffusers-hf/src/diffusers/models/upsampling.py:75-187 (nearest x2, optional 3x3 conv)."""

    def __init__(self, channels, use_conv=False, use_conv_transpose=False, out_channels=None):
        super().__init__()
        self.channels, self.out_channels = channels, out_channels or channels
        self.use_conv, self.use_conv_transpose = use_conv, use_conv_transpose
        self.conv = None
        if use_conv_transpose:
            self.conv = nn.ConvTranspose2d(channels, self.out_channels, 4, 2, 1)
        elif use_conv:
            self.conv = nn.Conv2d(channels, self.out_channels, 3, padding=1)

    def forward(self, x, output_size=None):
        if self.use_conv_transpose:
            return self.conv(x)
        if output_size is None:
            x = F.interpolate(x, scale_factor=2.0, mode="nearest")
        else:
            x = F.interpolate(x, size=output_size, mode="nearest")
        if self.use_conv:
            x = self.conv(x)
        return x


class ResnetBlock2D(nn.Module):
    """diffusers-hf/src/diffusers/models/resnet.py:222-415 (time_embedding_norm="default")."""

    def __init__(self, *, in_channels, out_channels=None, temb_channels=512, groups=32, eps=1e-6,
                 output_scale_factor=1.0, use_in_shortcut=None, up=False, down=False):
        super().__init__()
        out_channels = in_channels if out_channels is None else out_channels
        self.in_channels, self.out_channels = in_channels, out_channels
        self.output_scale_factor = output_scale_factor
        self.norm_silu1 = nn.Sequential(*fused_norm_silu(in_channels, groups, eps))
        self.conv1 = nn.Conv2d(in_channels, out_channels, 3, stride=1, padding=1)
        self.time_emb_proj = nn.Linear(temb_channels, out_channels) if temb_channels is not None else None
        self.norm_silu2 = nn.Sequential(*fused_norm_silu(out_channels, groups, eps))
        self.conv2 = nn.Conv2d(out_channels, out_channels, 3, stride=1, padding=1)
        self.upsample = self.downsample = None
        if up:
            self.upsample = Upsample2D(in_channels, use_conv=False)
        elif down:
            self.downsample = Downsample2D(in_channels, use_conv=False, padding=1, name="op")
        self.use_in_shortcut = in_channels != out_channels if use_in_shortcut is None else use_in_shortcut
        self.conv_shortcut = nn.Conv2d(in_channels, out_channels, 1) if self.use_in_shortcut else None

    def forward(self, input_tensor, temb):
        h = self.norm_silu1(input_tensor)
        if self.upsample is not None:
            input_tensor, h = self.upsample(input_tensor), self.upsample(h)
        elif self.downsample is not None:
            input_tensor, h = self.downsample(input_tensor), self.downsample(h)
        h = self.conv1(h)
        if self.time_emb_proj is not None:
            h = h + self.time_emb_proj(F.silu(temb))[:, :, None, None]
        h = self.norm_silu2(h)
        h = self.conv2(h)
        if self.conv_shortcut is not None:
            input_tensor = self.conv_shortcut(input_tensor)
        return (input_tensor + h) / self.output_scale_factor


# ----------------------------------------------------------------------------------- attention
class Attention(nn.Module):
    """diffusers-hf/src/diffusers/models/attention_processor.py:91-210 (constructor order to_q, to_k,
    to_v, to_out) with the AttnProcessor2_0 forward of :1219-1296."""

    def __init__(self, query_dim, cross_attention_dim=None, heads=8, dim_head=64, bias=False, out_bias=True):
        super().__init__()
        inner = heads * dim_head
        self.heads = heads
        kv_dim = cross_attention_dim if cross_attention_dim is not None else query_dim
        self.to_q = OracleLoRALinear(query_dim, inner, bias=bias)
        self.to_k = OracleLoRALinear(kv_dim, inner, bias=bias)
        self.to_v = OracleLoRALinear(kv_dim, inner, bias=bias)
        self.to_out = nn.ModuleList([OracleLoRALinear(inner, query_dim, bias=out_bias), nn.Dropout(0.0)])

    def forward(self, hidden_states, encoder_hidden_states=None):
        ctx = hidden_states if encoder_hidden_states is None else encoder_hidden_states
        q, k, v = self.to_q(hidden_states), self.to_k(ctx), self.to_v(ctx)
        o = O.attention(q, k, v, self.heads)
        return self.to_out[0](o)


class GEGLU(nn.Module):
    """diffusers-hf/src/diffusers/models/activations.py:111-149, unfused branch (single `proj`)."""

    def __init__(self, dim_in, dim_out):
        super().__init__()
        self.proj = OracleLoRALinear(dim_in, dim_out * 2)

    def forward(self, x):
        return O.geglu(self.proj(x))


class FeedForward(nn.Module):
    """diffusers-hf/src/diffusers/models/attention.py:608-664 (geglu, mult 4)."""

    def __init__(self, dim, mult=4):
        super().__init__()
        inner = dim * mult
        self.net = nn.ModuleList([GEGLU(dim, inner), nn.Dropout(0.0), OracleLoRALinear(inner, dim)])

    def forward(self, x):
        return self.net[2](self.net[0](x))


class BasicTransformerBlock(nn.Module):
    """diffusers-hf/src/diffusers/models/attention.py:124-403 with norm_type="layer_norm"."""

    def __init__(self, dim, num_attention_heads, attention_head_dim, cross_attention_dim=None):
        super().__init__()
        self.norm1 = nn.LayerNorm(dim, eps=1e-5)
        self.attn1 = Attention(dim, None, num_attention_heads, attention_head_dim)
        if cross_attention_dim is not None:
            self.norm2 = nn.LayerNorm(dim, eps=1e-5)
            self.attn2 = Attention(dim, cross_attention_dim, num_attention_heads, attention_head_dim)
        else:
            self.norm2 = self.attn2 = None
        self.norm3 = nn.LayerNorm(dim, eps=1e-5)
        self.ff = FeedForward(dim)

    def forward(self, h, encoder_hidden_states=None):
        h = self.attn1(self.norm1(h)) + h
        if self.attn2 is not None:
            h = self.attn2(self.norm2(h), encoder_hidden_states) + h
        return self.ff(self.norm3(h)) + h


class Transformer2DModel(nn.Module):
    """Continuous-input variant, diffusers-hf/src/diffusers/models/transformers/transformer_2d.py:172-207
    (constructor), :327-477, :479-492, :514-527 (forward)."""

    def __init__(self, num_attention_heads=16, attention_head_dim=88, in_channels=None, num_layers=1,
                 cross_attention_dim=None, norm_num_groups=32, use_linear_projection=False):
        super().__init__()
        inner = num_attention_heads * attention_head_dim
        self.use_linear_projection = use_linear_projection
        self.norm = nn.GroupNorm(norm_num_groups, in_channels, eps=1e-6, affine=True)
        if use_linear_projection:
            self.proj_in = OracleLoRALinear(in_channels, inner)
        else:
            self.proj_in = nn.Conv2d(in_channels, inner, 1)
        self.transformer_blocks = nn.ModuleList(
            [BasicTransformerBlock(inner, num_attention_heads, attention_head_dim, cross_attention_dim)
             for _ in range(num_layers)])
        if use_linear_projection:
            self.proj_out = OracleLoRALinear(inner, in_channels)
        else:
            self.proj_out = nn.Conv2d(inner, in_channels, 1)

    def forward(self, hidden_states, encoder_hidden_states=None):
        B, C, H, W = hidden_states.shape
        residual = hidden_states
        h = self.norm(hidden_states)
        if not self.use_linear_projection:
            h = self.proj_in(h)
            inner = h.shape[1]
            h = h.permute(0, 2, 3, 1).reshape(B, H * W, inner)
        else:
            inner = h.shape[1]
            h = h.permute(0, 2, 3, 1).reshape(B, H * W, inner)
            h = self.proj_in(h)
        for blk in self.transformer_blocks:
            h = blk(h, encoder_hidden_states)
        if not self.use_linear_projection:
            h = h.reshape(B, H, W, inner).permute(0, 3, 1, 2).contiguous()
            h = self.proj_out(h)
        else:
            h = self.proj_out(h)
            h = h.reshape(B, H, W, inner).permute(0, 3, 1, 2).contiguous()
        return h + residual


# ----------------------------------------------------------------------------------- UNet blocks
def _as_list(v, n):
    return [v] * n if isinstance(v, int) else list(v)


class DownBlock2D(nn.Module):
    """diffusers-hf/src/diffusers/models/unets/unet_2d_blocks.py:1303-1392."""

    has_cross_attention = False

    def __init__(self, in_channels, out_channels, temb_channels, num_layers=1, resnet_eps=1e-6, resnet_groups=32,
                 add_downsample=True, downsample_padding=1):
        super().__init__()
        self.resnets = nn.ModuleList([
            ResnetBlock2D(in_channels=in_channels if i == 0 else out_channels, out_channels=out_channels,
                          temb_channels=temb_channels, eps=resnet_eps, groups=resnet_groups)
            for i in range(num_layers)])
        self.downsamplers = nn.ModuleList([Downsample2D(out_channels, use_conv=True, out_channels=out_channels,
                                                        padding=downsample_padding, name="op")]) if add_downsample else None

    def forward(self, hidden_states, temb=None, encoder_hidden_states=None):
        outs = ()
        for resnet in self.resnets:
            hidden_states = resnet(hidden_states, temb)
            outs += (hidden_states,)
        if self.downsamplers is not None:
            hidden_states = self.downsamplers[0](hidden_states)
            outs += (hidden_states,)
        return hidden_states, outs


class CrossAttnDownBlock2D(nn.Module):
    """diffusers-hf/src/diffusers/models/unets/unet_2d_blocks.py:1140-1300."""

    has_cross_attention = True

    def __init__(self, in_channels, out_channels, temb_channels, num_layers=1, transformer_layers_per_block=1,
                 resnet_eps=1e-6, resnet_groups=32, num_attention_heads=1, cross_attention_dim=1280,
                 add_downsample=True, downsample_padding=1, use_linear_projection=False):
        super().__init__()
        tl = _as_list(transformer_layers_per_block, num_layers)
        resnets, attns = [], []
        for i in range(num_layers):
            resnets.append(ResnetBlock2D(in_channels=in_channels if i == 0 else out_channels, out_channels=out_channels,
                                         temb_channels=temb_channels, eps=resnet_eps, groups=resnet_groups))
            attns.append(Transformer2DModel(num_attention_heads, out_channels // num_attention_heads,
                                            in_channels=out_channels, num_layers=tl[i],
                                            cross_attention_dim=cross_attention_dim, norm_num_groups=resnet_groups,
                                            use_linear_projection=use_linear_projection))
        self.attentions = nn.ModuleList(attns)
        self.resnets = nn.ModuleList(resnets)
        self.downsamplers = nn.ModuleList([Downsample2D(out_channels, use_conv=True, out_channels=out_channels,
                                                        padding=downsample_padding, name="op")]) if add_downsample else None

    def forward(self, hidden_states, temb=None, encoder_hidden_states=None):
        outs = ()
        for resnet, attn in zip(self.resnets, self.attentions):
            hidden_states = resnet(hidden_states, temb)
            hidden_states = attn(hidden_states, encoder_hidden_states)
            outs += (hidden_states,)
        if self.downsamplers is not None:
            hidden_states = self.downsamplers[0](hidden_states)
            outs += (hidden_states,)
        return hidden_states, outs


class UNetMidBlock2DCrossAttn(nn.Module):
    """diffusers-hf/src/diffusers/models/unets/unet_2d_blocks.py:744-890."""

    has_cross_attention = True

    def __init__(self, in_channels, temb_channels, num_layers=1, transformer_layers_per_block=1, resnet_eps=1e-6,
                 resnet_groups=32, num_attention_heads=1, cross_attention_dim=1280, use_linear_projection=False):
        super().__init__()
        tl = _as_list(transformer_layers_per_block, num_layers)
        mk = lambda: ResnetBlock2D(in_channels=in_channels, out_channels=in_channels, temb_channels=temb_channels,
                                   eps=resnet_eps, groups=resnet_groups)
        resnets, attns = [mk()], []
        for i in range(num_layers):
            attns.append(Transformer2DModel(num_attention_heads, in_channels // num_attention_heads,
                                            in_channels=in_channels, num_layers=tl[i],
                                            cross_attention_dim=cross_attention_dim, norm_num_groups=resnet_groups,
                                            use_linear_projection=use_linear_projection))
            resnets.append(mk())
        self.attentions = nn.ModuleList(attns)
        self.resnets = nn.ModuleList(resnets)

    def forward(self, hidden_states, temb=None, encoder_hidden_states=None):
        hidden_states = self.resnets[0](hidden_states, temb)
        for attn, resnet in zip(self.attentions, self.resnets[1:]):
            hidden_states = attn(hidden_states, encoder_hidden_states)
            hidden_states = resnet(hidden_states, temb)
        return hidden_states


class UpBlock2D(nn.Module):
    """diffusers-hf/src/diffusers/models/unets/unet_2d_blocks.py:2558-2670."""

    has_cross_attention = False

    def __init__(self, in_channels, prev_output_channel, out_channels, temb_channels, num_layers=1, resnet_eps=1e-6,
                 resnet_groups=32, add_upsample=True):
        super().__init__()
        resnets = []
        for i in range(num_layers):
            res_skip = in_channels if (i == num_layers - 1) else out_channels
            res_in = prev_output_channel if i == 0 else out_channels
            resnets.append(ResnetBlock2D(in_channels=res_in + res_skip, out_channels=out_channels,
                                         temb_channels=temb_channels, eps=resnet_eps, groups=resnet_groups))
        self.resnets = nn.ModuleList(resnets)
        self.upsamplers = nn.ModuleList([Upsample2D(out_channels, use_conv=True, out_channels=out_channels)]) if add_upsample else None

    def forward(self, hidden_states, res_hidden_states_tuple, temb=None, encoder_hidden_states=None):
        for resnet in self.resnets:
            res = res_hidden_states_tuple[-1]
            res_hidden_states_tuple = res_hidden_states_tuple[:-1]
            hidden_states = torch.cat([hidden_states, res], dim=1)
            hidden_states = resnet(hidden_states, temb)
        if self.upsamplers is not None:
            hidden_states = self.upsamplers[0](hidden_states)
        return hidden_states


class CrossAttnUpBlock2D(nn.Module):
    """diffusers-hf/src/diffusers/models/unets/unet_2d_blocks.py:2382-2555."""

    has_cross_attention = True

    def __init__(self, in_channels, out_channels, prev_output_channel, temb_channels, num_layers=1,
                 transformer_layers_per_block=1, resnet_eps=1e-6, resnet_groups=32, num_attention_heads=1,
                 cross_attention_dim=1280, add_upsample=True, use_linear_projection=False):
        super().__init__()
        tl = _as_list(transformer_layers_per_block, num_layers)
        resnets, attns = [], []
        for i in range(num_layers):
            res_skip = in_channels if (i == num_layers - 1) else out_channels
            res_in = prev_output_channel if i == 0 else out_channels
            resnets.append(ResnetBlock2D(in_channels=res_in + res_skip, out_channels=out_channels,
                                         temb_channels=temb_channels, eps=resnet_eps, groups=resnet_groups))
            attns.append(Transformer2DModel(num_attention_heads, out_channels // num_attention_heads,
                                            in_channels=out_channels, num_layers=tl[i],
                                            cross_attention_dim=cross_attention_dim, norm_num_groups=resnet_groups,
                                            use_linear_projection=use_linear_projection))
        self.attentions = nn.ModuleList(attns)
        self.resnets = nn.ModuleList(resnets)
        self.upsamplers = nn.ModuleList([Upsample2D(out_channels, use_conv=True, out_channels=out_channels)]) if add_upsample else None

    def forward(self, hidden_states, res_hidden_states_tuple, temb=None, encoder_hidden_states=None):
        for resnet, attn in zip(self.resnets, self.attentions):
            res = res_hidden_states_tuple[-1]
            res_hidden_states_tuple = res_hidden_states_tuple[:-1]
            hidden_states = torch.cat([hidden_states, res], dim=1)
            hidden_states = resnet(hidden_states, temb)
            hidden_states = attn(hidden_states, encoder_hidden_states)
        if self.upsamplers is not None:
            hidden_states = self.upsamplers[0](hidden_states)
        return hidden_states
