"""Closed forms of the hot-path operators, CPU fp32/fp64 (checker for the HIP kernels).

Pinned by tests/test_oracle_ops.py: merge identity, scale-0, adapter order independence, brute-force
fp64 loops on tiny shapes, torch library routines (F.group_norm, F.layer_norm, F.gelu,
F.scaled_dot_product_attention).
"""
from __future__ import annotations

import math
from typing import Optional, Sequence

import torch
import torch.nn.functional as F


def lora_linear(x, weight, bias=None, adapters: Sequence[tuple] = (), residual=None):
    """y = x W^T + b + sum_i s_i * (x A_i^T) B_i^T.

    adapters: sequence of (A_i [r,in], B_i [out,r], s_i) with s_i the complete multiplier
    (adapter weight * alpha / rank * global scale).
    Base + scale * (up(down(x))): diffusers-hf/src/diffusers/models/lora.py:451-457 (LoRACompatibleLinear.forward)
    with the low-rank branch of :222-232 (LoRALinearLayer.forward; alpha/rank at :227-228).
    """
    y = F.linear(x, weight, bias)
    for A, B, s in adapters:
        y = y + float(s) * F.linear(F.linear(x, A), B)
    if residual is not None:
        y = y + residual
    return y


def lora_merged_weight(weight, adapters: Sequence[tuple]):
    """W + sum_i s_i * B_i A_i -- the fused-weight form.

    diffusers: w_orig + lora_scale * bmm(w_up, w_down) (diffusers-hf/src/diffusers/models/lora.py:409-425);
    Katz: unet_weight += (up @ down) * (alpha / rank) (diffusers-hf/src/diffusers/pipelines/controlnet/
    pipeline_controlnet_sd_xl_katz.py:1737-1747).
    """
    w = weight.clone()
    for A, B, s in adapters:
        w = w + float(s) * (B @ A)
    return w


def lora_conv2d(x, weight, bias=None, adapters: Sequence[tuple] = (), stride: int = 1, padding: int = 1):
    """conv(x, W) + sum_i s_i * conv1x1(conv_k(x, A_i), B_i) with A_i [r, in, k, k], B_i [out, r, 1, 1] (or [out, r]).

    LoRACompatibleConv.forward (diffusers-hf/src/diffusers/models/lora.py:369-383) + LoRAConv2dLayer.forward
    (:284-296): the down conv has the base conv's kernel, stride and padding, the up conv is 1x1;
    s_i = weight_i * alpha_i / rank_i.  Equal to the conv with the merged kernel of _fuse_lora (:403-421):
    W + s * (B.flatten(1) @ A.flatten(1)).reshape(W.shape)."""
    y = F.conv2d(x, weight, bias, stride=stride, padding=padding)
    for A, B, s in adapters:
        t = F.conv2d(x, A, None, stride=stride, padding=padding)
        y = y + float(s) * F.conv2d(t, B.reshape(B.shape[0], B.shape[1], 1, 1))
    return y


def attention(q, k, v, heads: int, scale: Optional[float] = None):
    """softmax(q k^T * scale) v per head, inputs [B,T,H*d] / [B,S,H*d], output [B,T,H*d].

    Follows AttnProcessor2_0.__call__: view to [B,h,T,d] (diffusers-hf/src/diffusers/models/
    attention_processor.py:1269-1272), F.scaled_dot_product_attention without mask or dropout (:1276-1278),
    heads merged back (:1280).  Written out explicitly (not through SDPA) so SDPA can pin it.
    """
    B, T, inner = q.shape
    S = k.shape[1]
    d = inner // heads
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    qh = q.view(B, T, heads, d).transpose(1, 2)
    kh = k.view(B, S, heads, d).transpose(1, 2)
    vh = v.view(B, S, heads, d).transpose(1, 2)
    p = torch.softmax((qh @ kh.transpose(-1, -2)) * scale, dim=-1)
    return (p @ vh).transpose(1, 2).reshape(B, T, inner)


def group_norm(x, num_groups: int, weight, bias, eps: float, activation: str = "none"):
    """GroupNorm over [N,C,H,W] followed by an optional SiLU.

    The reference's fused op (diffusers-hf/src/diffusers/models/normalization.py:79-103 calling
    fast_kernel group_norm_fp16 with "silu") replaces nn.GroupNorm + nn.SiLU (:36-37; the original
    two-op form is kept in the comments at diffusers-hf/src/diffusers/models/resnet.py:363-365).
    Statistics per (sample, group) over (C/G)*H*W elements, biased variance
    (diffusers-hf/src/fast_kernel/fast_kernel/csrc/normalize.cuh:207-301 Welford).
    """
    N, C = x.shape[:2]
    xg = x.reshape(N, num_groups, -1)
    mean = xg.mean(dim=2, keepdim=True)
    var = xg.var(dim=2, unbiased=False, keepdim=True)
    y = ((xg - mean) * torch.rsqrt(var + eps)).reshape(x.shape)
    if weight is not None:
        y = y * weight.view(1, C, *([1] * (x.dim() - 2)))
    if bias is not None:
        y = y + bias.view(1, C, *([1] * (x.dim() - 2)))
    if activation == "silu":
        y = y * torch.sigmoid(y)
    elif activation != "none":
        raise ValueError(activation)
    return y


def layer_norm(x, weight, bias, eps: float = 1e-5):
    """nn.LayerNorm over the last axis (diffusers-hf/src/diffusers/models/attention.py:195,225,253)."""
    mean = x.mean(dim=-1, keepdim=True)
    var = x.var(dim=-1, unbiased=False, keepdim=True)
    y = (x - mean) * torch.rsqrt(var + eps)
    if weight is not None:
        y = y * weight
    if bias is not None:
        y = y + bias
    return y


def gelu(x, approximate: str = "none"):
    """erf-exact or tanh GELU (diffusers-hf/src/diffusers/models/activations.py:133-137;
    tanh form diffusers-hf/src/fast_kernel/fast_kernel/csrc/gelu.cuh:29-42)."""
    if approximate == "tanh":
        return 0.5 * x * (1.0 + torch.tanh(0.7978845608028654 * (x + 0.044715 * x * x * x)))
    return 0.5 * x * (1.0 + torch.erf(x * 0.7071067811865476))


def geglu(proj, approximate: str = "none"):
    """hidden, gate = proj.chunk(2, -1); hidden * gelu(gate)
    (diffusers-hf/src/diffusers/models/activations.py:148-149)."""
    h, g = proj.chunk(2, dim=-1)
    return h * gelu(g, approximate)


def gelu_mul(x, m, approximate: str = "tanh"):
    """gelu(x) * m: fast_gelu_mul_fp16(x, m) (diffusers-hf/src/fast_kernel/fast_kernel/csrc/gelu.cuh:36-41),
    called as fast_gelu_mul(proj_2(x), proj_1(x)) at activations.py:145."""
    return gelu(x, approximate) * m


def residual_mean(residual_sets: Sequence[torch.Tensor]):
    """Multi-ControlNet reduce: sum then divide by the count
    (diffusers-hf/src/diffusers/models/unets/unet_2d_condition.py:1424-1439)."""
    acc = residual_sets[0].clone()
    for r in residual_sets[1:]:
        acc = acc + r
    return acc / len(residual_sets)


def residual_add(dst, residual_sets: Sequence[torch.Tensor]):
    """skip_j + r_j / sample + r_mid (unet_2d_condition.py:1284-1292)."""
    return dst + residual_mean(residual_sets)


def concat_residual(h, skip, residual_sets: Sequence[torch.Tensor] = ()):
    """torch.cat([h, skip + r], dim=1): the residual add of unet_2d_condition.py:1284-1290 followed by
    the up-block concat (diffusers-hf/src/diffusers/models/unets/unet_2d_blocks.py:2512)."""
    s = residual_add(skip, residual_sets) if len(residual_sets) else skip
    return torch.cat([h, s], dim=1)


def sgmv(x, seg_start: Sequence[int], seg_adapter: Sequence[int], adapters: Sequence[tuple], y_base):
    """Per-request adapters: rows of segment s get y += s_a (x A_a^T) B_a^T -- lora_linear applied
    request by request (the reference has no batched form)."""
    y = y_base.clone()
    for s, a in enumerate(seg_adapter):
        if a < 0:
            continue
        r0, r1 = seg_start[s], seg_start[s + 1]
        A, B, sc = adapters[a]
        y[r0:r1] = y[r0:r1] + float(sc) * F.linear(F.linear(x[r0:r1], A), B)
    return y
