"""Host-side layers of the adapter-augmented SDXL UNet, running on the katz_hip kernels.

Module, attribute and state-dict names are the reference's (Katz fork of diffusers 0.28):
`norm_silu1.0`, `to_q/to_k/to_v/to_out.0`, `ff.net.0.proj`, `ff.net.2`, `proj_in/proj_out`, ... so
checkpoints and LoRA key maps written for the reference address these modules unchanged.

Activations are bf16.  4-D feature maps are torch tensors of shape [N,C,H,W] in channels_last memory
(NHWC): the convolutions (MIOpen) take and return that format, GroupNorm reads it directly, and the
token view [N, H*W, C] the transformer blocks need is the same memory -- the NCHW<->token permute +
.contiguous() copies of the reference (transformer_2d.py:488-490, :516-518) do not exist here.
"""
from __future__ import annotations

import os
from typing import Dict, List, Optional, Sequence

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops
from .lora import (MAX_PACKED_RANK, Adapter, PackedAdapters, fold_layer_norm, interleave_geglu_rows, pack_adapters,
                   rescale_)

CL = torch.channels_last


# When True, LoRALinear leaves its weights uninitialised (for models whose state dict is loaded next).
SKIP_INIT = False

# How a LoRALinear with active adapters runs:
#   "fused": one launch, the rank-R product is computed per output tile and kept in LDS;
#   "split": kh_lora_shrink_bf16 once per layer input, then the base GEMM + expand reading it from L2.
LORA_MODE = os.getenv("KATZ_LORA_MODE", "split")
# split mode: "in_launch" lets kh_lora_linear_split_bf16 run the shrink inside the GEMM launch where the GEMM leaves
# CUs idle; "separate" always makes two launches (for measurements)
LORA_SHRINK = os.getenv("KATZ_LORA_SHRINK", "in_launch")

# The three LayerNorms of a transformer block (attention.py:338-403) are folded into the projections behind them: the
# linear that produces the hidden states leaves per-row sums, the linear that consumes the norm's output reads the
# un-normalised rows and finishes the normalisation in its epilogue (kh_lora_linear_norm_bf16).  "0": run every
# LayerNorm as a kernel of its own (for measurements).
LN_FOLD = os.getenv("KATZ_LN_FOLD", "1") != "0"

# A cross-attention over a short context (the 77 text tokens) runs inside the epilogue of its query projection where the
# projection's 128 x 128 tiles fill at most one round of CUs (kh_lora_linear_xattn_bf16).  "0": projection, then the
# attention kernel (for measurements).
XATTN_FUSE = os.getenv("KATZ_XATTN_FUSE", "1") != "0"

# The 3x3 convolutions of a residual block leave the statistics of the GroupNorm behind them as a by-product of their
# epilogue (kh_conv3x3_gn_stats_nhwc_bf16), so that norm is one launch instead of two.  "0": convolution, then the norm's
# two launches (for measurements).
CONV_GN_FUSE = os.getenv("KATZ_CONV_GN_FUSE", "1") != "0"


class RowStats:
    """Per-row (sum, sum of squares) partials of the current hidden states of a transformer, written by the linear
    that produced them (`valid`), read by the linear behind the next LayerNorm."""

    def __init__(self, M: int, device):
        self.buf = ops.row_stats_buffer(M, device)
        self.valid = False


# bumped whenever any layer rebuilds its packed adapter buffers (not on pure scale changes): consumers
# that cache pointers into those buffers (grouped launches) rebuild when it moves
_pack_epoch = 0


class LoRALinear(nn.Module):
    """nn.Linear whose forward is the fused base-GEMM + low-rank-delta kernel.

    Equivalent of the peft `Linear` wrapper the reference injects
    (diffusers-hf/src/diffusers/loaders/lora.py:409,475-476) and of LoRACompatibleLinear
    (diffusers-hf/src/diffusers/models/lora.py:386-457): named adapters, an active list, per-adapter
    weights, a global scale, fuse / unfuse.  geglu=True fuses GEGLU.forward's chunk + gelu + mul
    (diffusers-hf/src/diffusers/models/activations.py:148-149) into the epilogue.
    """

    def __init__(self, in_features: int, out_features: int, bias: bool = True, geglu: bool = False,
                 device=None, dtype=None):
        super().__init__()
        self.in_features, self.out_features, self.geglu = in_features, out_features, geglu
        self.weight = nn.Parameter(torch.empty((out_features, in_features), device=device, dtype=dtype), requires_grad=False)
        self.bias = nn.Parameter(torch.empty(out_features, device=device, dtype=dtype), requires_grad=False) if bias else None
        self.adapters: Dict[str, Adapter] = {}
        self.active: List[str] = []
        self.global_scale = 1.0
        self.adapters_enabled = True
        self._packed: Optional[PackedAdapters] = None
        self._packed_key = None
        self._rt = None          # (weight version, weight ptr, runtime weight, runtime bias)
        self._ln_rt = None       # (key, folded operands) for the LayerNorm in front of this layer
        self._fused: Dict[str, float] = {}   # adapter name -> multiplier merged into weight
        self.reset_parameters()

    def reset_parameters(self):
        if self.weight.device.type != "meta" and not SKIP_INIT:
            lin = nn.Linear(self.in_features, self.out_features, bias=self.bias is not None)
            with torch.no_grad():
                self.weight.copy_(lin.weight)
                if self.bias is not None:
                    self.bias.copy_(lin.bias)

    # ---- adapter state (host) ---------------------------------------------------------------
    def add_adapter(self, name: str, down: torch.Tensor, up: torch.Tensor, alpha: Optional[float] = None,
                    weight: float = 1.0) -> None:
        if down.shape[1] != self.in_features or up.shape[0] != self.out_features or down.shape[0] != up.shape[1]:
            raise ValueError(f"adapter {name!r} does not fit a [{self.out_features},{self.in_features}] layer: "
                             f"down {tuple(down.shape)}, up {tuple(up.shape)}")
        self.adapters[name] = Adapter(down.detach(), up.detach(), alpha, weight)
        self._packed_key = None

    def delete_adapter(self, name: str) -> None:
        self.adapters.pop(name, None)
        self.active = [n for n in self.active if n != name]
        self._packed_key = None

    def set_active(self, names: Sequence[str], weights: Optional[Sequence[float]] = None) -> None:
        self.active = [n for n in names if n in self.adapters]
        if weights is not None:
            for n, w in zip(names, weights):
                if n in self.adapters:
                    self.adapters[n].weight = float(w)
        self.refresh_adapters()

    def set_global_scale(self, scale: float) -> None:
        """cross_attention_kwargs["scale"]: scale_lora_layers, diffusers-hf/src/diffusers/utils/peft_utils.py:103-123."""
        if scale != self.global_scale:
            self.global_scale = float(scale)
            self.refresh_adapters()

    def refresh_adapters(self) -> None:
        """(Re)build the packed buffers; a pure scale change only rewrites col_scale in place, so a
        captured HIP graph that reads the buffers stays valid."""
        global _pack_epoch
        names = [n for n in self.active if n not in self._fused] if self.adapters_enabled else []
        key = tuple((n, id(self.adapters[n].down)) for n in names)
        if not names:
            if self._packed is not None:
                _pack_epoch += 1
            self._packed, self._packed_key = None, key
            return
        if key == self._packed_key and self._packed is not None:
            rescale_(self._packed, self.adapters, self.global_scale)
            return
        # more than 128 rank columns: the extra packs are applied one by one after the fused launch (forward), which for
        # a GEGLU projection means before the activation, so everything is packed in the plain row order then
        wide = sum(self.adapters[n].rank for n in names) > MAX_PACKED_RANK
        self._packed = pack_adapters(self.adapters, names, self.in_features, self.out_features, self.weight.dtype,
                                     self.weight.device, self.global_scale, geglu_interleave=self.geglu and not wide)
        self._packed_key = key
        _pack_epoch += 1

    def fuse(self, lora_scale: float = 1.0, names: Optional[Sequence[str]] = None) -> None:
        """W += sum_i (lora_scale * m_i) B_i A_i in fp32, cast back -- _fuse_lora,
        diffusers-hf/src/diffusers/models/lora.py:403-433 (Katz: pipeline_controlnet_sd_xl_katz.py:1737-1747)."""
        names = list(self.active if names is None else names)
        merged = self._fuse_candidate(lora_scale, names)
        if merged is not None:
            self._fuse_commit(*merged)

    def _fuse_candidate(self, lora_scale: float, names: Sequence[str]):
        """(merged fp32 weight, {adapter: multiplier}) without touching any state, or None when there is nothing to
        fuse.  Raises if the merged weight is not finite: like the reference (lora.py:416-421) the layer is then left
        exactly as it was."""
        todo = {}
        with torch.no_grad():
            w = self.weight.float()
            dev = self.weight.device
            for n in names:
                if n in self._fused or n in todo or n not in self.adapters:
                    continue
                ad = self.adapters[n]
                m = lora_scale * ad.multiplier(1.0)
                w = w + m * (ad.up.to(dev).float() @ ad.down.to(dev).float())
                todo[n] = m
            if not todo:
                return None
            if not torch.isfinite(w).all():
                raise ValueError("fusing produced non-finite weights; LoRA left unfused")
        return w, todo

    def _fuse_commit(self, w: torch.Tensor, todo: Dict[str, float]) -> None:
        with torch.no_grad():
            self.weight.copy_(w.to(self.weight.dtype))
        self._fused.update(todo)
        self.refresh_adapters()

    def unfuse(self) -> None:
        with torch.no_grad():
            w = self.weight.float()
            dev = self.weight.device
            for n, m in self._fused.items():
                ad = self.adapters[n]
                w = w - m * (ad.up.to(dev).float() @ ad.down.to(dev).float())
            self.weight.copy_(w.to(self.weight.dtype))
        self._fused.clear()
        self.refresh_adapters()

    # ---- runtime -----------------------------------------------------------------------------------
    def prepare(self) -> None:
        """Build the kernel-side weight buffers (the GEGLU row interleave) for the current weights."""
        ver = (self.weight._version, self.weight.data_ptr(), None if self.bias is None else self.bias._version)
        if self._rt is not None and self._rt[0] == ver:
            return
        if self.geglu:
            w = interleave_geglu_rows(self.weight.detach())
            b = interleave_geglu_rows(self.bias.detach()) if self.bias is not None else None
        else:
            w = self.weight.detach()
            b = self.bias.detach() if self.bias is not None else None
        self._rt = (ver, w, b)
        self._packed_key = None  # weights moved or changed: repack on their device / dtype
        self.refresh_adapters()

    def norm_path_ok(self, x: torch.Tensor, stats: bool = False) -> bool:
        """Can this call go through kh_lora_linear_norm_bf16 (a folded LayerNorm in front, row statistics out)?"""
        p = self._packed
        return (LN_FOLD and x.dtype == torch.bfloat16 and self.weight.dtype == torch.bfloat16 and self.in_features % 64 == 0
                and self.out_features % 8 == 0 and (p is None or (not p.overflow and LORA_MODE == "split"))
                and (not stats or (self.out_features <= 128 * ops.LN_SLOTS and not self.geglu)))

    def _ln_terms(self, norm: "LayerNorm"):
        """(W', c1, c2, A', ca1, ca2) of this layer behind `norm` (lora.fold_layer_norm), rebuilt when the weights, the
        norm's parameters or the packed adapters change."""
        _, w, b = self._rt
        p = self._packed
        key = (self._rt[0], id(norm), norm.weight._version, norm.bias._version, norm.weight.data_ptr(),
               None if p is None else (p.a_cat.data_ptr(), p.a_cat._version))
        if self._ln_rt is None or self._ln_rt[0] != key:
            self._ln_rt = (key, fold_layer_norm(w, b, norm.weight, norm.bias, None if p is None else p.a_cat))
        return self._ln_rt[1]

    def forward(self, x: torch.Tensor, residual: Optional[torch.Tensor] = None, ln=None,
                stats_out: Optional[RowStats] = None) -> torch.Tensor:
        """ln = (LayerNorm module, RowStats of x): the layer computes on norm(x); with valid statistics the norm is folded
        into the GEMM, otherwise it runs as a kernel of its own.  stats_out: left describing the result (valid) when the
        layer can write them, marked invalid otherwise."""
        self.prepare()
        _, w, b = self._rt
        p = self._packed
        fold = ln is not None and ln[1] is not None and ln[1].valid and self.norm_path_ok(x)
        emit = stats_out is not None and self.norm_path_ok(x, stats=True) and not (fold and ln[1] is stats_out)
        if ln is not None and not fold:
            x = ln[0](x)
        if fold or emit:
            a = s = bc = lnarg = None
            r_used = 0
            if p is not None:
                a, s, bc, r_used = p.a_cat, p.col_scale, p.b_cat, p.r_used
            if fold:
                norm, st = ln
                w, c1, c2, ap, ca1, ca2 = self._ln_terms(norm)
                b = None
                a = ap if p is not None else None
                lnarg = (st.buf, c1, c2, ca1, ca2, norm.eps)
            y = ops.lora_linear_norm(x, w, b, a, s, bc, residual=residual, geglu=self.geglu,
                                     two_launches=LORA_SHRINK == "separate", r_used=r_used, ln=lnarg,
                                     stats_out=stats_out.buf if emit else None)
            if stats_out is not None:
                stats_out.valid = emit
            return y
        if stats_out is not None:
            stats_out.valid = False
        if p is None:
            return ops.lora_linear(x, w, b, residual=residual, geglu=self.geglu)
        if p.overflow:
            return self._forward_wide(x, residual, p)
        if LORA_MODE == "split" and x.dtype == torch.bfloat16 and self.in_features % 64 == 0:
            return ops.lora_linear_split(x, w, b, p.a_cat, p.col_scale, p.b_cat, residual=residual, geglu=self.geglu,
                                         two_launches=LORA_SHRINK == "separate", r_used=p.r_used)
        return ops.lora_linear(x, w, b, p.a_cat, p.b_cat, p.col_scale, residual=residual, geglu=self.geglu)

    def forward_attention(self, x: torch.Tensor, k: torch.Tensor, v: torch.Tensor, heads: int, scale: float, ln=None):
        """This layer as the query projection of an attention over k / v [B,S,heads*64]: softmax(q k^T * scale) v with
        q = forward(x, ln=ln), in one launch where the kernel takes the shapes (ops.lora_linear_xattn); None otherwise
        (the caller then runs forward and the attention kernel)."""
        if not XATTN_FUSE or x.dim() != 3 or not x.is_cuda or x.dtype != torch.bfloat16 or self.geglu:
            return None
        self.prepare()
        _, w, b = self._rt
        p = self._packed
        B, T, K = x.shape
        R = 0 if p is None else p.R
        if w.dtype != torch.bfloat16 or (p is not None and (p.overflow or LORA_MODE != "split")):
            return None
        if k.shape != (B, k.shape[1], self.out_features) or v.shape != k.shape or k.stride(-1) != 1 or v.stride(-1) != 1:
            return None
        if not ops.lora_linear_xattn_ok(B * T, self.out_features, K, R, T, k.shape[1], heads):
            return None
        a = sc = bc = lnarg = None
        r_used = 0
        if p is not None:
            a, sc, bc, r_used = p.a_cat, p.col_scale, p.b_cat, p.r_used
        if ln is not None:
            if ln[1] is not None and ln[1].valid and self.norm_path_ok(x):
                norm, st = ln
                w, c1, c2, ap, ca1, ca2 = self._ln_terms(norm)
                b = None
                a = ap if p is not None else None
                lnarg = (st.buf, c1, c2, ca1, ca2, norm.eps)
            else:
                x = ln[0](x)
        return ops.lora_linear_xattn(x, w, k, v, heads, scale, bias=b, a_cat=a, col_scale=sc, b_cat=bc,
                                     two_launches=LORA_SHRINK == "separate", r_used=r_used, ln=lnarg)

    def _forward_wide(self, x, residual, p: PackedAdapters) -> torch.Tensor:
        """More rank columns than one launch takes (sum of the active ranks > 128; peft has no such limit): the first
        128 go with the base GEMM, every further pack adds ((x A^T) * scale) B^T with y as the residual of a GEMM over
        its rank columns.  A GEGLU projection is computed in the reference's row order without the fused epilogue and
        activated afterwards (all packs belong under the activation)."""
        w = self.weight.detach() if self.geglu else self._rt[1]
        b = (None if self.bias is None else self.bias.detach()) if self.geglu else self._rt[2]
        y = ops.lora_linear(x, w, b, p.a_cat, p.b_cat, p.col_scale, residual=None if self.geglu else residual)
        for c in p.overflow:
            t = ops.lora_linear(x, c.a_cat, None)                       # [.., R] = x A^T
            t.mul_(c.col_scale.to(t.dtype))
            y = ops.lora_linear(t, c.b_cat, None, residual=y)
        if self.geglu:
            return ops.geglu(y)
        return y

    def extra_repr(self) -> str:
        return f"in_features={self.in_features}, out_features={self.out_features}, bias={self.bias is not None}, geglu={self.geglu}"


class GroupNorm(nn.Module):
    """GroupNorm with the activation fused, replacing the reference's
    diffusers-hf/src/diffusers/models/normalization.py:40-103 (fast_kernel group_norm_fp16)."""

    def __init__(self, num_groups: int, num_channels: int, eps: float = 1e-5, affine: bool = True,
                 activation: str = "none", device=None, dtype=None):
        super().__init__()
        self.num_groups, self.num_channels, self.eps, self.activation = num_groups, num_channels, eps, activation
        if affine:
            self.weight = nn.Parameter(torch.ones(num_channels, device=device, dtype=dtype), requires_grad=False)
            self.bias = nn.Parameter(torch.zeros(num_channels, device=device, dtype=dtype), requires_grad=False)
        else:
            self.weight = self.bias = None

    def forward(self, x: torch.Tensor, add_nc: Optional[torch.Tensor] = None) -> torch.Tensor:
        st = getattr(x, "_katz_gn_stats", None)
        if (st is not None and CONV_GN_FUSE and st.num_groups == self.num_groups and st.version == x._version
                and st.add_nc is add_nc and (self.weight is None or self.weight.dtype == torch.bfloat16)):
            # the convolution that produced x left this norm's statistics (Conv3x3.forward, stats_for): one launch
            return ops.group_norm_from_stats(x, self.num_groups, self.weight, self.bias, self.eps, self.activation,
                                             st.partials, st.splits, add_nc=add_nc)
        return ops.group_norm(x, self.num_groups, self.weight, self.bias, self.eps, self.activation, add_nc=add_nc)


class GnStats:
    """GroupNorm statistics that ride on a convolution's output tensor (attribute `_katz_gn_stats`) to the norm behind it:
    partial (sum, sum of squares) per (image, group, row tile) of the tensor + add_nc, valid while the tensor's version
    counter has not moved."""
    __slots__ = ("partials", "splits", "num_groups", "add_nc", "version")

    def __init__(self, partials, splits, num_groups, add_nc, version):
        self.partials, self.splits, self.num_groups, self.add_nc, self.version = partials, splits, num_groups, add_nc, version


def fused_norm_silu(num_channels: int, norm_num_groups: int, eps: float, affine: bool = True):
    """One fused module where the reference returns [GroupNorm(activation fused)] under
    ENABLE_FUSED_NORM_SILU=1 (normalization.py:30-35): keeps the `<name>.0.weight` state-dict keys."""
    return [GroupNorm(norm_num_groups, num_channels, eps=eps, affine=affine, activation="silu")]


class LayerNorm(nn.Module):
    def __init__(self, dim: int, eps: float = 1e-5, device=None, dtype=None):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim, device=device, dtype=dtype), requires_grad=False)
        self.bias = nn.Parameter(torch.zeros(dim, device=device, dtype=dtype), requires_grad=False)

    def forward(self, x):
        return ops.layer_norm(x, self.weight, self.bias, self.eps)


class TimestepEmbedding(nn.Module):
    """linear_1 -> SiLU -> linear_2 on [B, C] (two rows: not worth a custom kernel)."""

    def __init__(self, in_channels: int, time_embed_dim: int):
        super().__init__()
        self.linear_1 = nn.Linear(in_channels, time_embed_dim)
        self.linear_2 = nn.Linear(time_embed_dim, time_embed_dim)

    def forward(self, sample):
        return self.linear_2(F.silu(self.linear_1(sample)))


class _ConvLoRAFuse:
    """W += sum_i (lora_scale * m_i) * (up_i . down_i) for a convolution, through the merged-kernel identity of the
    reference: the [Cout, r] x [r, Cin*kh*kw] product reshaped to the weight's shape (_fuse_lora of LoRACompatibleConv,
    diffusers-hf/src/diffusers/models/lora.py:403-421; _unfuse_lora :423-441), fp32 then cast back.  Shared by the 3x3
    and the 1x1 convolution; same all-or-nothing contract as LoRALinear.fuse."""

    def _delta(self, ad: Adapter, m: float) -> torch.Tensor:
        dev = self.weight.device
        up = ad.up.to(dev).float().reshape(ad.up.shape[0], -1)
        down = ad.down.to(dev).float().reshape(ad.down.shape[0], -1)
        return (m * (up @ down)).reshape(self.weight.shape)

    def _fuse_candidate(self, lora_scale: float, names: Sequence[str]):
        todo = {}
        with torch.no_grad():
            w = self.weight.float()
            for n in names:
                if n in self._fused or n in todo or n not in self.adapters:
                    continue
                m = lora_scale * self.adapters[n].multiplier(1.0)
                w = w + self._delta(self.adapters[n], m)
                todo[n] = m
            if not todo:
                return None
            if not torch.isfinite(w).all():
                raise ValueError("fusing produced non-finite weights; LoRA left unfused")
        return w, todo

    def _fuse_commit(self, w: torch.Tensor, todo: Dict[str, float]) -> None:
        with torch.no_grad():
            self.weight.copy_(w.to(self.weight.dtype))
        self._fused.update(todo)
        self.refresh_adapters()

    def fuse(self, lora_scale: float = 1.0, names: Optional[Sequence[str]] = None) -> None:
        merged = self._fuse_candidate(lora_scale, list(self.active if names is None else names))
        if merged is not None:
            self._fuse_commit(*merged)

    def unfuse(self) -> None:
        if not self._fused:
            return
        with torch.no_grad():
            w = self.weight.float()
            for n, m in self._fused.items():
                w = w - self._delta(self.adapters[n], m)
            self.weight.copy_(w.to(self.weight.dtype))
        self._fused.clear()
        self.refresh_adapters()


class Conv3x3(_ConvLoRAFuse, nn.Conv2d):
    """nn.Conv2d(kernel 3, padding 1, stride 1 or 2) whose forward runs the katz_hip implicit-GEMM kernel on
    channels_last bf16 GPU tensors; parameters and state-dict keys are nn.Conv2d's.  forward(x, residual)
    also folds the residual add that follows the convolution (resnet.py:374) into the kernel's epilogue.
    Channel counts the kernel does not take directly (the 4-channel latent, the 3-channel conditioning image) are
    zero-padded; other dtypes / devices / paddings run torch's conv2d."""

    def __init__(self, in_channels, out_channels, stride=1, padding=1):
        super().__init__(in_channels, out_channels, 3, stride=stride, padding=padding)
        self._packed = None  # (weight data_ptr, weight version, [Cout,3,3,Cin] copy)
        # LoRA on the convolution (LoRACompatibleConv + LoRAConv2dLayer, diffusers-hf/src/diffusers/models/lora.py
        # :258-296, :369-383): down [r,Cin,3,3] with the base conv's stride / padding, up [Cout,r,1,1]
        self.adapters: Dict[str, Adapter] = {}
        self.active: List[str] = []
        self.adapters_enabled = True
        self._global_scale = 1.0
        self._lora = None    # (A_cat packed [R,3,3,Cin], B_cat scaled [Cout,R]) of the active adapters
        self._fused: Dict[str, float] = {}   # adapter name -> multiplier merged into weight

    def add_adapter(self, name: str, down: torch.Tensor, up: torch.Tensor, alpha: Optional[float] = None,
                    weight: float = 1.0) -> None:
        up = up.reshape(up.shape[0], up.shape[1])
        if down.dim() != 4 or tuple(down.shape[1:]) != (self.in_channels, 3, 3) or up.shape != (self.out_channels, down.shape[0]):
            raise ValueError(f"adapter {name!r}: expected down [r,{self.in_channels},3,3] and up [{self.out_channels},r(,1,1)], "
                             f"got {tuple(down.shape)} and {tuple(up.shape)}")
        self.adapters[name] = Adapter(down.detach(), up.detach(), alpha, weight)
        self._lora = None

    def delete_adapter(self, name: str) -> None:
        self.adapters.pop(name, None)
        self.active = [n for n in self.active if n != name]
        self._lora = None

    def set_active(self, names: Sequence[str], weights: Optional[Sequence[float]] = None) -> None:
        self.active = [n for n in names if n in self.adapters]
        if weights is not None:
            for n, w in zip(names, weights):
                if n in self.adapters:
                    self.adapters[n].weight = float(w)
        self._lora = None

    def set_global_scale(self, scale: float) -> None:
        if scale != self._global_scale:
            self._global_scale = float(scale)
            self._lora = None

    def refresh_adapters(self) -> None:
        self._lora = None

    def _lora_pack(self):
        """A_cat: the active down kernels stacked along the rank axis, zero-padded to a multiple of 32, in the conv
        kernel's [R,3,3,Cin] layout; B_cat [Cout,R] with each adapter's weight * alpha / rank * global scale folded in."""
        if self._lora is None:
            names = [n for n in self.active if self.adapters_enabled and n not in self._fused]
            if not names:
                self._lora = (None, None)
            else:
                dev, dt = self.weight.device, self.weight.dtype
                downs = [self.adapters[n].down.to(dev, torch.float32) for n in names]
                ups = [self.adapters[n].up.to(dev, torch.float32) * self.adapters[n].multiplier(self._global_scale) for n in names]
                a = torch.cat(downs, dim=0)
                b = torch.cat(ups, dim=1)
                pad = -a.shape[0] % 32
                a = F.pad(a, (0, 0, 0, 0, 0, -self.in_channels % 32, 0, pad))
                b = F.pad(b, (0, pad))
                self._lora = (ops.pack_conv3x3_weight(a.to(dt)), b.to(dt).contiguous())
        return self._lora

    def packed_weight(self):
        """([Cout', 3, 3, Cin'] weight, [Cout'] bias) in the kernel's layout, channel counts zero-padded up to what
        the kernel takes (Cin' % 32 == 0, Cout' % 8 == 0): padded input channels meet zero weights, padded output
        channels are dropped by the caller."""
        w = self.weight
        if self._packed is None or self._packed[0] != w.data_ptr() or self._packed[1] != w._version:
            pi, po = -self.in_channels % 32, -self.out_channels % 8
            wp = w.detach()
            b = None if self.bias is None else self.bias.detach()
            if pi or po:
                wp = F.pad(wp, (0, 0, 0, 0, 0, pi, 0, po))
                b = None if b is None else F.pad(b, (0, po))
            self._packed = (w.data_ptr(), w._version, ops.pack_conv3x3_weight(wp), b)
        return self._packed[2], self._packed[3]

    def forward(self, x, residual=None, stats_for=None):
        """stats_for = (num_groups, add_nc or None): a GroupNorm of that many groups follows (on the result + add_nc per image
        and channel); where the kernel takes the shape the convolution's epilogue leaves its statistics, which ride on
        the returned tensor (GnStats) and make that norm one launch instead of two."""
        native = (x.is_cuda and x.dtype == torch.bfloat16 and self.weight.dtype == torch.bfloat16 and self.padding == (1, 1))
        a_cat, b_cat = self._lora_pack() if self.adapters else (None, None)
        if (stats_for is not None and CONV_GN_FUSE and native and a_cat is None and self.in_channels % 32 == 0
                and self.out_channels % 8 == 0):
            groups, add_nc = stats_for
            add_ok = add_nc is None or (add_nc.dtype == torch.bfloat16 and add_nc.numel() == x.shape[0] * self.out_channels
                                        and add_nc.is_contiguous())
            if add_ok and ops.conv3x3_gn_splits(x, self.out_channels, groups, self.stride[0]) > 0:
                x = x.contiguous(memory_format=torch.channels_last)
                if residual is not None:
                    residual = residual.contiguous(memory_format=torch.channels_last)
                w_packed, b_packed = self.packed_weight()
                y, partials, splits = ops.conv3x3_stats(x, w_packed, b_packed, groups, add_nc=add_nc, residual=residual,
                                                        stride=self.stride[0])
                y._katz_gn_stats = GnStats(partials, splits, groups, add_nc, y._version)
                return y
        if not native:
            if a_cat is not None:
                raise NotImplementedError("LoRA on a convolution needs the katz_hip conv kernel (bf16 GPU tensors, padding 1)")
            y = super().forward(x)
            return y if residual is None else residual + y
        pi, po = -self.in_channels % 32, -self.out_channels % 8
        if pi:   # few-channel inputs (the latent, the conditioning image): zero channels up to the kernel's granule
            x = F.pad(x, (0, 0, 0, 0, 0, pi))
        x = x.contiguous(memory_format=torch.channels_last)   # no copy when the producer already wrote NHWC
        w_packed, b_packed = self.packed_weight()
        if po:
            if a_cat is not None:
                raise NotImplementedError("LoRA on a convolution whose output channels are not a multiple of 8")
            y = ops.conv3x3(x, w_packed, b_packed, stride=self.stride[0])[:, :self.out_channels]
            y = y.contiguous(memory_format=torch.channels_last)
            return y if residual is None else residual + y
        if residual is not None:
            residual = residual.contiguous(memory_format=torch.channels_last)
        y = ops.conv3x3(x, w_packed, b_packed, stride=self.stride[0], residual=residual)
        if a_cat is None:
            return y
        # low-rank branch: T = conv3x3(x, A_cat) is [pixels, R]; y += T . B_cat^T as a GEMM with y as its residual
        t = ops.conv3x3(x, a_cat, None, stride=self.stride[0])
        nb, co, ho, wo = y.shape
        y2 = ops.lora_linear(t.permute(0, 2, 3, 1).reshape(nb * ho * wo, t.shape[1]), b_cat, None,
                             residual=y.permute(0, 2, 3, 1).reshape(nb * ho * wo, co))
        return y2.view(nb, ho, wo, co).permute(0, 3, 1, 2)


class Conv1x1(_ConvLoRAFuse, nn.Conv2d):
    """1x1 convolution (the resnets' conv_shortcut) with the reference's LoRA on it: down [r,Cin,1,1], up [Cout,r,1,1]
    (LoRAConv2dLayer, diffusers-hf/src/diffusers/models/lora.py:258-296; LoRACompatibleConv.forward :369-383).  On
    channels_last bf16 GPU tensors it is a linear layer over the channels of every pixel and runs on the LoRA linear
    kernel, adapters included; parameters and state-dict keys are nn.Conv2d's."""

    def __init__(self, in_channels, out_channels):
        super().__init__(in_channels, out_channels, 1)
        self.adapters: Dict[str, Adapter] = {}
        self.active: List[str] = []
        self.adapters_enabled = True
        self._global_scale = 1.0
        self._packed = None       # PackedAdapters of the active adapters, False = none active
        self._fused: Dict[str, float] = {}

    def add_adapter(self, name: str, down: torch.Tensor, up: torch.Tensor, alpha: Optional[float] = None,
                    weight: float = 1.0) -> None:
        r = down.shape[0]
        if down.numel() != r * self.in_channels or up.numel() != self.out_channels * r or up.shape[0] != self.out_channels:
            raise ValueError(f"adapter {name!r}: expected down [r,{self.in_channels}(,1,1)] and up [{self.out_channels},r(,1,1)], "
                             f"got {tuple(down.shape)} and {tuple(up.shape)}")
        self.adapters[name] = Adapter(down.detach().reshape(r, self.in_channels), up.detach().reshape(self.out_channels, r),
                                      alpha, weight)
        self._packed = None

    def delete_adapter(self, name: str) -> None:
        self.adapters.pop(name, None)
        self.active = [n for n in self.active if n != name]
        self._packed = None

    def set_active(self, names: Sequence[str], weights: Optional[Sequence[float]] = None) -> None:
        self.active = [n for n in names if n in self.adapters]
        if weights is not None:
            for n, w in zip(names, weights):
                if n in self.adapters:
                    self.adapters[n].weight = float(w)
        self._packed = None

    def set_global_scale(self, scale: float) -> None:
        if scale != self._global_scale:
            self._global_scale = float(scale)
            self._packed = None

    def refresh_adapters(self) -> None:
        self._packed = None

    def _pack(self):
        if self._packed is None:
            names = [n for n in self.active if self.adapters_enabled and n not in self._fused]
            self._packed = pack_adapters(self.adapters, names, self.in_channels, self.out_channels, self.weight.dtype,
                                         self.weight.device, self._global_scale) if names else False
        return self._packed or None

    def forward(self, x):
        if not (x.is_cuda and x.dtype == torch.bfloat16 and self.weight.dtype == torch.bfloat16
                and self.in_channels % 32 == 0 and self.out_channels % 8 == 0):
            if self.adapters and self.active:
                raise NotImplementedError("LoRA on a 1x1 convolution needs the katz_hip kernels (bf16 GPU tensors)")
            return super().forward(x)
        x = x.contiguous(memory_format=torch.channels_last)
        nb, c, hh, ww = x.shape
        p = self._pack() if self.adapters else None
        x2 = x.permute(0, 2, 3, 1).reshape(nb * hh * ww, c)
        w2 = self.weight.reshape(self.out_channels, c)
        if p is None:
            y = ops.lora_linear(x2, w2, self.bias)
        else:
            y = ops.lora_linear(x2, w2, self.bias, p.a_cat, p.b_cat, p.col_scale)
            for c in p.overflow:      # rank columns beyond the 128 one launch takes (see LoRALinear._forward_wide)
                t = ops.lora_linear(x2, c.a_cat, None)
                t.mul_(c.col_scale.to(t.dtype))
                y = ops.lora_linear(t, c.b_cat, None, residual=y)
        return y.view(nb, hh, ww, self.out_channels).permute(0, 3, 1, 2)


class Downsample2D(nn.Module):
    def __init__(self, channels, use_conv=True, out_channels=None, padding=1, name="op", stats_groups=None):
        """stats_groups: the number of groups of the GroupNorm that reads the result next (the following block's first
        resnet); its statistics then ride on the output (see Conv3x3.forward)."""
        super().__init__()
        self.padding = padding
        self.stats_groups = stats_groups
        self.conv = Conv3x3(channels, out_channels or channels, stride=2, padding=padding)

    def forward(self, x):
        if self.padding == 0:
            x = F.pad(x, (0, 1, 0, 1))
        return self.conv(x, stats_for=None if self.stats_groups is None else (self.stats_groups, None))


class Upsample2D(nn.Module):
    def __init__(self, channels, use_conv=True, out_channels=None):
        super().__init__()
        self.conv = Conv3x3(channels, out_channels or channels)

    def forward(self, x, output_size=None):
        if output_size is None:
            if (x.is_cuda and x.dtype == torch.bfloat16 and x.shape[1] % 8 == 0
                    and x.is_contiguous(memory_format=torch.channels_last)):
                x = ops.upsample_nearest2x(x)
            else:
                x = F.interpolate(x, scale_factor=2.0, mode="nearest")
        else:
            x = F.interpolate(x, size=output_size, mode="nearest")
        return self.conv(x)


class ResnetBlock2D(nn.Module):
    """diffusers-hf/src/diffusers/models/resnet.py:352-415 with both GroupNorm+SiLU pairs on the fused kernel."""

    def __init__(self, *, in_channels, out_channels=None, temb_channels=512, groups=32, eps=1e-6,
                 output_scale_factor=1.0):
        super().__init__()
        out_channels = in_channels if out_channels is None else out_channels
        self.output_scale_factor = output_scale_factor
        self.norm_silu1 = nn.Sequential(*fused_norm_silu(in_channels, groups, eps))
        self.conv1 = Conv3x3(in_channels, out_channels)
        self.time_emb_proj = nn.Linear(temb_channels, out_channels)
        self.norm_silu2 = nn.Sequential(*fused_norm_silu(out_channels, groups, eps))
        self.conv2 = Conv3x3(out_channels, out_channels)
        self.conv_shortcut = Conv1x1(in_channels, out_channels) if in_channels != out_channels else None
        self.temb_proj = None   # this step's time_emb_proj(temb_act), when a TimeEmbProjector computed it ahead

    def forward(self, input_tensor, temb_act):
        """temb_act = silu(temb), computed once per step by the caller."""
        h = self.norm_silu1(input_tensor)
        # hidden_states + temb[:, :, None, None] rides inside the second norm (no separate pass), and where the kernel takes
        # the shape conv1's epilogue leaves that norm's statistics (they ride on conv1's output tensor)
        tp, self.temb_proj = self.temb_proj, None
        add = self.time_emb_proj(temb_act) if tp is None else tp
        norm2 = self.norm_silu2[0]
        h = norm2(self.conv1(h, stats_for=(norm2.num_groups, add)), add_nc=add)
        if self.conv_shortcut is not None:
            input_tensor = self.conv_shortcut(input_tensor)
        # input_tensor + conv2(h), the add in the conv's epilogue; what follows a resnet is mostly another GroupNorm (the
        # transformer's, the next resnet's, conv_norm_out) with this block's number of groups: its statistics ride along
        out = self.conv2(h, residual=input_tensor, stats_for=(norm2.num_groups, None))
        if self.output_scale_factor != 1.0:
            out = out / self.output_scale_factor
        return out


class TimeEmbProjector:
    """time_emb_proj(silu(temb)) of EVERY resnet of the model at the start of the step, one batched launch per output
    width instead of one two-row GEMM per resnet inside the chain of big kernels (the reference computes each where
    it is used, resnet.py:381-390).  Same arithmetic, same inputs; nothing is kept across steps."""

    def __init__(self, resnets: Sequence["ResnetBlock2D"]):
        self.groups: Dict[int, List[ResnetBlock2D]] = {}
        for r in resnets:
            self.groups.setdefault(r.time_emb_proj.out_features, []).append(r)
        self._stacked: Dict[int, tuple] = {}   # width -> (key, W [G,C,K], b [G,1,C])

    @staticmethod
    def _key(rs):
        return tuple((r.time_emb_proj.weight.data_ptr(), r.time_emb_proj.weight._version, r.time_emb_proj.bias._version)
                     for r in rs)

    def run(self, temb_act: torch.Tensor) -> None:
        for width, rs in self.groups.items():
            key = self._key(rs)
            st = self._stacked.get(width)
            if st is None or st[0] != key:
                if temb_act.is_cuda and torch.cuda.is_current_stream_capturing():
                    raise RuntimeError("katz_amd: run the step once eagerly before capturing it (stacked time_emb_proj weights)")
                with torch.no_grad():
                    w = torch.stack([r.time_emb_proj.weight.detach() for r in rs]).contiguous()
                    b = torch.stack([r.time_emb_proj.bias.detach() for r in rs]).unsqueeze(1).contiguous()
                st = (key, w, b)
                self._stacked[width] = st
            _, w, b = st
            x = temb_act.to(w.dtype).unsqueeze(0).expand(len(rs), -1, -1)
            y = torch.baddbmm(b, x, w.transpose(1, 2))          # [G, N, C], every resnet's [N, C] contiguous
            for i, r in enumerate(rs):
                r.temb_proj = y[i]


class KatzAttnProcessor:
    """Attention processor on the katz_hip flash kernel; plugs into the reference's processor API
    (Attention.set_processor, attention_processor.py:374-392; call signature :1219-1228).
    q/k/v stay in the projection layout [B, tokens, heads*64]; `residual` (optional) is added inside
    the to_out projection's epilogue."""

    def __call__(self, attn, hidden_states, encoder_hidden_states=None, attention_mask=None, temb=None,
                 residual=None, ln=None, stats_out=None, **kwargs):
        """ln = (LayerNorm module, RowStats): hidden_states are the input of that norm, which is folded into the query
        (self-attention: q/k/v) projection; stats_out: a RowStats the output projection fills (see LoRALinear.forward)."""
        if attention_mask is not None:
            raise NotImplementedError("attention masks are not used on the SDXL path and not implemented")
        qkv = attn.fused_qkv(hidden_states, ln=ln) if encoder_hidden_states is None else None
        if qkv is None and ln is not None and encoder_hidden_states is None:
            hidden_states, ln = ln[0](hidden_states), None   # three separate projections: normalise once
        ctx = hidden_states if encoder_hidden_states is None else encoder_hidden_states
        if qkv is not None:
            q, k, v = qkv  # self-attention: one shrink + one GEMM for the three projections
        elif encoder_hidden_states is not None and attn.ctx_kv is not None and attn.ctx_kv[0] is encoder_hidden_states:
            _, k, v = attn.ctx_kv  # projected for every cross-attention at once at the start of the step
        else:
            k = attn.to_k(ctx)
            v = attn.to_v(ctx)
        o = None
        if qkv is None:
            # a short context: the attention runs inside the query projection's launch where the kernel takes the shapes
            if encoder_hidden_states is not None:
                o = attn.to_q.forward_attention(hidden_states, k, v, attn.heads, attn.scale, ln=ln)
            if o is None:
                q = attn.to_q(hidden_states, ln=ln)
        if o is None:
            o = ops.attention(q, k, v, attn.heads, attn.scale)
        o = attn.to_out[0](o, residual=residual, stats_out=stats_out)
        return attn.to_out[1](o)


class Attention(nn.Module):
    """diffusers-hf/src/diffusers/models/attention_processor.py:91-210, :484-525."""

    def __init__(self, query_dim, cross_attention_dim=None, heads=8, dim_head=64, bias=False, out_bias=True,
                 processor=None):
        super().__init__()
        inner = heads * dim_head
        self.heads, self.scale = heads, dim_head ** -0.5
        kv_dim = cross_attention_dim if cross_attention_dim is not None else query_dim
        self.to_q = LoRALinear(query_dim, inner, bias=bias)
        self.to_k = LoRALinear(kv_dim, inner, bias=bias)
        self.to_v = LoRALinear(kv_dim, inner, bias=bias)
        self.to_out = nn.ModuleList([LoRALinear(inner, query_dim, bias=out_bias), nn.Dropout(0.0)])
        self.processor = processor or KatzAttnProcessor()
        self.is_cross = cross_attention_dim is not None
        self.ctx_kv = None  # (context tensor, k, v) filled by ContextKVProjector for the current step
        self._qkv = None    # fused to_q/to_k/to_v state (self-attention only)

    def fused_qkv(self, x: torch.Tensor, ln=None):
        """to_q / to_k / to_v of a self-attention as ONE GEMM over the stacked weights ([3N,K]: three
        times the workgroups of a single projection, which alone covers 160 of 256 CUs) and, with
        adapters, ONE shrink over the stacked A matrices.  Returns (q, k, v) as column views of the
        [.., 3N] result, or None when the layers cannot be fused (then they run one by one)."""
        layers = (self.to_q, self.to_k, self.to_v)
        N, K = self.to_q.out_features, self.to_q.in_features
        if self.is_cross or x.dtype != torch.bfloat16 or N % 128 != 0 or K % 64 != 0:
            return None
        for l in layers:
            l.prepare()
        sig = (_pack_epoch, tuple((l.weight.data_ptr(), l.weight._version) for l in layers), LORA_MODE)
        st = self._qkv
        if st is None or st["sig"] != sig:
            packs = [l._packed for l in layers]
            same = all(p is None for p in packs) or (all(p is not None and not p.overflow for p in packs) and len({p.R for p in packs}) == 1)
            ok = same and (packs[0] is None or LORA_MODE == "split") and all(l.bias is None for l in layers)
            st = dict(sig=sig, ok=ok)
            if ok:
                st["w"] = torch.cat([l.weight.detach() for l in layers], dim=0).contiguous()
                st["R"] = 0 if packs[0] is None else packs[0].R
                if st["R"]:
                    R = st["R"]
                    st["r_used"] = max(p.r_used for p in packs)
                    st["a"] = torch.cat([p.a_cat for p in packs], dim=0).contiguous()
                    st["s"] = torch.cat([p.col_scale for p in packs], dim=0).contiguous()
                    st["b"] = torch.cat([p.b_cat for p in packs], dim=0).contiguous()
                    for g, p in enumerate(packs):  # the layers now read (and rescale) the stacked storage
                        p.a_cat, p.col_scale = st["a"][g * R:(g + 1) * R], st["s"][g * R:(g + 1) * R]
            self._qkv = st
        if not st["ok"]:
            return None
        if ln is not None and ln[1] is not None and ln[1].valid and LN_FOLD:
            # the norm in front is folded into the stacked GEMM (ln = (LayerNorm, RowStats of x))
            norm, stats = ln
            key = (id(norm), norm.weight._version, norm.bias._version, norm.weight.data_ptr())
            if st.get("ln_key") != key:
                st["ln"] = fold_layer_norm(st["w"], None, norm.weight, norm.bias, st["a"] if st["R"] else None)
                st["ln_key"] = key
            wp, c1, c2, ap, ca1, ca2 = st["ln"]
            y = ops.lora_linear_norm(x, wp, None, ap, st["s"] if st["R"] else None, st["b"] if st["R"] else None,
                                     two_launches=LORA_SHRINK == "separate", n_split=N if st["R"] else 0,
                                     r_used=st["r_used"] if st["R"] else 0, ln=(stats.buf, c1, c2, ca1, ca2, norm.eps))
            return y.split(N, dim=-1)
        if ln is not None:
            x = ln[0](x)
        if st["R"]:
            y = ops.lora_linear_split(x, st["w"], None, st["a"], st["s"], st["b"], n_split=N,
                                      two_launches=LORA_SHRINK == "separate", r_used=st["r_used"])
        else:
            y = ops.lora_linear(x, st["w"], None)
        return y.split(N, dim=-1)

    def set_processor(self, processor) -> None:
        self.processor = processor

    def get_processor(self):
        return self.processor

    def forward(self, hidden_states, encoder_hidden_states=None, attention_mask=None, **cross_attention_kwargs):
        return self.processor(self, hidden_states, encoder_hidden_states=encoder_hidden_states,
                              attention_mask=attention_mask, **cross_attention_kwargs)


def env_flag(name: str) -> bool:
    """The reference's switches are environment variables read when a module is built, "1" = on
    (ENABLE_FUSED_GEGLU diffusers-hf/src/diffusers/models/activations.py:123, ENABLE_FUSED_NORM_SILU
    normalization.py:31, ENABLE_CHANNELS_LAST resnet.py:330, ENABLE_CUDA_GRAPH unets/unet_2d_condition.py:511)."""
    import os

    return os.getenv(name, "0") == "1"


class GEGLU(nn.Module):
    """`proj` holds the reference's [2*inner, dim] weight (value rows then gate rows); the kernel reads a
    row-interleaved copy and applies value * gelu(gate) in the GEMM epilogue.

    ENABLE_FUSED_GEGLU=1 (read at construction, like activations.py:123) selects the arithmetic of the reference's
    fused op instead: value * gelu_tanh(gate) (fast_gelu_mul_fp16(proj_2(x), proj_1(x)), activations.py:145,
    csrc/gelu.cuh:29-42) -- the projection then runs without the epilogue and kh_geglu_bf16 applies the tanh form.
    Off (the default) is the exact erf form of the unfused branch (:148-149)."""

    def __init__(self, dim_in, dim_out):
        super().__init__()
        self.enable_fused_geglu = env_flag("ENABLE_FUSED_GEGLU")
        self.proj = LoRALinear(dim_in, dim_out * 2, geglu=not self.enable_fused_geglu)

    def forward(self, x, ln=None):
        if self.enable_fused_geglu:
            return ops.geglu(self.proj(x, ln=ln), approximate="tanh")
        return self.proj(x, ln=ln)


class FeedForward(nn.Module):
    def __init__(self, dim, mult=4):
        super().__init__()
        inner = dim * mult
        self.net = nn.ModuleList([GEGLU(dim, inner), nn.Dropout(0.0), LoRALinear(inner, dim)])

    def forward(self, x, residual=None, ln=None, stats_out=None):
        return self.net[2](self.net[0](x, ln=ln), residual=residual, stats_out=stats_out)


class BasicTransformerBlock(nn.Module):
    """diffusers-hf/src/diffusers/models/attention.py:283-403 (layer_norm variant); the three residual
    adds run in the epilogues of to_out.0 (x2) and ff.net.2."""

    def __init__(self, dim, num_attention_heads, attention_head_dim, cross_attention_dim=None):
        super().__init__()
        self.norm1 = LayerNorm(dim, 1e-5)
        self.attn1 = Attention(dim, None, num_attention_heads, attention_head_dim)
        if cross_attention_dim is not None:
            self.norm2 = LayerNorm(dim, 1e-5)
            self.attn2 = Attention(dim, cross_attention_dim, num_attention_heads, attention_head_dim)
        else:
            self.norm2 = self.attn2 = None
        self.norm3 = LayerNorm(dim, 1e-5)
        self.ff = FeedForward(dim)

    def forward(self, h, encoder_hidden_states=None, stats: Optional[RowStats] = None, last: bool = False):
        """stats: the row statistics of h as its producer left them (or invalid); on return they describe the result,
        unless `last` (nobody reads them).  Without it every norm runs as a kernel of its own."""
        if stats is None:
            h = self.attn1(self.norm1(h), residual=h)
            if self.attn2 is not None:
                h = self.attn2(self.norm2(h), encoder_hidden_states=encoder_hidden_states, residual=h)
            return self.ff(self.norm3(h), residual=h)
        h = self.attn1(h, ln=(self.norm1, stats), residual=h, stats_out=stats)
        if self.attn2 is not None:
            h = self.attn2(h, encoder_hidden_states=encoder_hidden_states, ln=(self.norm2, stats), residual=h, stats_out=stats)
        return self.ff(h, ln=(self.norm3, stats), residual=h, stats_out=None if last else stats)


class Transformer2DModel(nn.Module):
    """diffusers-hf/src/diffusers/models/transformers/transformer_2d.py:327-527, linear-projection variant
    (the only one SDXL uses).  Input / output: channels_last [N,C,H,W]."""

    def __init__(self, num_attention_heads, attention_head_dim, in_channels, num_layers=1, cross_attention_dim=None,
                 norm_num_groups=32, use_linear_projection=True):
        super().__init__()
        if not use_linear_projection:
            raise NotImplementedError("only use_linear_projection=True (SDXL) is implemented")
        inner = num_attention_heads * attention_head_dim
        self.norm = GroupNorm(norm_num_groups, in_channels, eps=1e-6, affine=True, activation="none")
        self.proj_in = LoRALinear(in_channels, inner)
        self.transformer_blocks = nn.ModuleList(
            [BasicTransformerBlock(inner, num_attention_heads, attention_head_dim, cross_attention_dim)
             for _ in range(num_layers)])
        self.proj_out = LoRALinear(inner, in_channels)

    def forward(self, hidden_states, encoder_hidden_states=None):
        N, C, H, W = hidden_states.shape
        tokens = lambda t: t.permute(0, 2, 3, 1).reshape(N, H * W, C)  # a view of channels_last memory
        residual = tokens(hidden_states)
        h = tokens(self.norm(hidden_states))
        stats = RowStats(N * H * W, h.device) if LN_FOLD and h.dtype == torch.bfloat16 else None
        h = self.proj_in(h, stats_out=stats)
        for i, blk in enumerate(self.transformer_blocks):
            h = blk(h, encoder_hidden_states, stats=stats, last=i + 1 == len(self.transformer_blocks))
        h = self.proj_out(h, residual=residual)
        return h.view(N, H, W, C).permute(0, 3, 1, 2)


class ContextKVProjector:
    """to_k / to_v of EVERY cross-attention of the model in one grouped launch per width.

    The text context is the same tensor for all 70 cross-attentions of a step, and each of their
    K/V projections is a 154-row GEMM that cannot fill 256 CUs on its own (the reference issues
    them one by one, attention_processor.py:1260-1262).  Here the 2 x 70 projections run as one launch
    per output width (grid.y = layer), and with adapters active one shrink launch computes
    context . A^T for all of them (their A matrices stacked).  The step's arithmetic is unchanged --
    nothing is cached across steps.
    """

    def __init__(self, attentions: Sequence["Attention"]):
        self.groups: Dict[int, List[Attention]] = {}
        for a in attentions:
            if a.is_cross:
                self.groups.setdefault(a.to_k.out_features, []).append(a)
        self._built = {}  # width -> dict(state)

    def _layers(self, width):
        out = []
        for a in self.groups[width]:
            out += [a.to_k, a.to_v]
        return out

    def _build(self, width: int, M: int, ctx: torch.Tensor):
        layers = self._layers(width)
        for l in layers:
            l.prepare()
        K = layers[0].in_features
        packs = [l._packed for l in layers]
        uniform = all(p is None for p in packs) or (all(p is not None and not p.overflow for p in packs) and len({p.R for p in packs}) == 1)
        ok = uniform and LORA_MODE == "split" and all(l.weight.dtype == torch.bfloat16 and not l.geglu for l in layers)
        st = dict(epoch=_pack_epoch, M=M, ok=ok, wptr=[l.weight.data_ptr() for l in layers])
        if ok:
            dev = ctx.device
            G = len(layers)
            R = 0 if packs[0] is None else packs[0].R
            y = torch.empty((G, M, width), dtype=torch.bfloat16, device=dev)
            t = a_all = s_all = None
            if R > 0:
                a_all = torch.cat([p.a_cat for p in packs], dim=0).contiguous()
                s_all = torch.cat([p.col_scale for p in packs], dim=0).contiguous()
                for g, p in enumerate(packs):  # the layers now read (and rescale) the stacked storage
                    p.a_cat = a_all[g * R:(g + 1) * R]
                    p.col_scale = s_all[g * R:(g + 1) * R]
                t = torch.empty((M, G * R), dtype=torch.bfloat16, device=dev)
            rows = []
            for g, l in enumerate(layers):
                _, w, b = l._rt
                rows.append([w.data_ptr(), 0 if b is None else b.data_ptr(), 0 if R == 0 else packs[g].b_cat.data_ptr(),
                             0 if R == 0 else t.data_ptr() + g * R * 2, y[g].data_ptr()])
            st.update(G=G, R=R, K=K, y=y, t=t, a_all=a_all, s_all=s_all,
                      table=torch.tensor(rows, dtype=torch.int64, device=dev))
        self._built[width] = st
        return st

    def run(self, ctx: torch.Tensor) -> None:
        """Project `ctx` [B,S,K] for every cross-attention; results are handed to the Attention modules."""
        B, S, K = ctx.shape
        M = B * S
        for width, attns in self.groups.items():
            st = self._built.get(width)
            layers = self._layers(width)
            if (st is None or st["epoch"] != _pack_epoch or st["M"] != M
                    or st["wptr"] != [l.weight.data_ptr() for l in layers]):
                st = self._build(width, M, ctx)
            if not st["ok"]:
                for a in attns:
                    a.ctx_kv = None
                continue
            x2 = ctx.reshape(M, K)
            if st["R"] > 0:
                ops.lora_shrink(x2, st["a_all"], st["s_all"], out=st["t"])
            ops.lora_linear_grouped(x2, st["table"], M, width, K, st["R"], st["G"] * st["R"] if st["R"] else 8)
            for i, a in enumerate(attns):
                a.ctx_kv = (ctx, st["y"][2 * i].view(B, S, width), st["y"][2 * i + 1].view(B, S, width))
