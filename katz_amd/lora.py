"""Host side of the LoRA surface: adapter registry per layer and the packed layout the kernels read.

The reference keeps one (lora_A, lora_B, alpha, rank, weight) set per adapter inside peft's Linear
wrappers and turns them on / off and scales them from the host
(set_weights_and_activate_adapters, diffusers-hf/src/diffusers/utils/peft_utils.py:238-269;
scale_lora_layers / unscale_lora_layers :103-147).  Here the ACTIVE adapters of a layer are packed
once per activation change into

    A_cat [R, in]   rows of all active A_i stacked, zero padded to R % 32 == 0
    B_cat [out, R]  columns of all active B_i side by side, zero padded
    col_scale [R]   fp32, weight_i * alpha_i / rank_i * global_scale for the columns of adapter i

so that sum_i s_i B_i A_i x is ONE rank-R product inside the fused kernel, and changing a scale only
rewrites col_scale.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import torch

RANK_PAD = 64   # packed rank is padded to the K-stage depth of the GEMM that consumes it
MAX_PACKED_RANK = 128


@dataclass
class Adapter:
    """One LoRA on one layer: down = lora_A [r, in], up = lora_B [out, r]
    (LoRALinearLayer.down/up, diffusers-hf/src/diffusers/models/lora.py:210-211)."""

    down: torch.Tensor
    up: torch.Tensor
    alpha: Optional[float] = None  # network_alpha; None means alpha == rank (lora.py:227-228)
    weight: float = 1.0            # set_adapters weight

    @property
    def rank(self) -> int:
        return self.down.shape[0]

    def multiplier(self, global_scale: float = 1.0) -> float:
        a = self.rank if self.alpha is None else self.alpha
        return float(self.weight) * float(a) / float(self.rank) * float(global_scale)


@dataclass
class PackedAdapters:
    a_cat: torch.Tensor
    b_cat: torch.Tensor
    col_scale: torch.Tensor
    spans: List[tuple] = field(default_factory=list)  # (name, first column, rank)
    # Rank columns beyond the kernels' 128: further packs of at most 128 columns each (A rows / B columns of the same
    # adapters, continued).  Only LoRALinear's own forward applies them; the fused launches that stack several
    # layers' packs take the per-layer path when a layer has any.
    overflow: List["PackedAdapters"] = field(default_factory=list)

    @property
    def R(self) -> int:
        return self.a_cat.shape[0]

    @property
    def r_used(self) -> int:
        """Rank columns that can be non-zero (the adapters' ranks side by side), rounded up to the 16 columns of one
        MFMA step; the columns from there to R are zero padding."""
        used = max((c + r for _, c, r in self.spans), default=0)
        return min(self.R, (used + 15) // 16 * 16)


def interleave_geglu_rows(t: torch.Tensor) -> torch.Tensor:
    """Reorder the output-feature axis (dim 0) of a GEGLU projection tensor from
    [value(0..D) | gate(0..D)] (hidden, gate = proj(x).chunk(2, -1),
    diffusers-hf/src/diffusers/models/activations.py:148) to blocks of 32 value rows followed by
    their 32 gate rows, the order the fused GEGLU epilogue consumes."""
    two_d = t.shape[0]
    D = two_d // 2
    if two_d % 64 != 0:
        raise ValueError("GEGLU interleave needs 2*D % 64 == 0")
    v = t[:D].reshape(D // 32, 1, 32, *t.shape[1:])
    g = t[D:].reshape(D // 32, 1, 32, *t.shape[1:])
    return torch.cat([v, g], dim=1).reshape(t.shape).contiguous()


def pack_adapters(adapters: Dict[str, Adapter], active: Sequence[str], in_features: int, out_features: int,
                  dtype, device, global_scale: float = 1.0, geglu_interleave: bool = False) -> Optional[PackedAdapters]:
    """Build A_cat / B_cat / col_scale for the active adapters (in the given order). Returns None when
    nothing is active (the layer then runs as a plain Linear, like peft with adapters disabled)."""
    names = [n for n in active if n in adapters]
    if not names:
        return None
    for n in names:
        ad = adapters[n]
        if ad.down.shape != (ad.rank, in_features) or ad.up.shape != (out_features, ad.rank):
            raise ValueError(f"adapter {n!r}: down {tuple(ad.down.shape)} / up {tuple(ad.up.shape)} do not fit "
                             f"a [{out_features},{in_features}] layer")
    total = sum(adapters[n].rank for n in names)
    if total > MAX_PACKED_RANK and geglu_interleave:
        raise ValueError("more than 128 rank columns on a GEGLU projection need the plain row order: pack with "
                         "geglu_interleave=False (LoRALinear does)")
    # cut the adapters' rank rows, in order, into packs of at most MAX_PACKED_RANK columns
    packs, pieces, width = [], [], 0
    for n in names:
        r, r0 = adapters[n].rank, 0
        while r0 < r:
            take = min(r - r0, MAX_PACKED_RANK - width)
            pieces.append((n, r0, take))
            width += take
            r0 += take
            if width == MAX_PACKED_RANK:
                packs.append(pieces)
                pieces, width = [], 0
    if pieces:
        packs.append(pieces)
    built = []
    for pcs in packs:
        used = sum(t for _, _, t in pcs)
        R = (used + RANK_PAD - 1) // RANK_PAD * RANK_PAD
        a_cat = torch.zeros((R, in_features), dtype=dtype, device=device)
        b_cat = torch.zeros((out_features, R), dtype=dtype, device=device)
        col_scale = torch.zeros((R,), dtype=torch.float32, device=device)
        spans, c = [], 0
        for n, r0, take in pcs:
            ad = adapters[n]
            a_cat[c:c + take] = ad.down[r0:r0 + take].to(device=device, dtype=dtype)
            b_cat[:, c:c + take] = ad.up[:, r0:r0 + take].to(device=device, dtype=dtype)
            col_scale[c:c + take] = ad.multiplier(global_scale)
            spans.append((n, c, take))
            c += take
        if geglu_interleave:
            b_cat = interleave_geglu_rows(b_cat)
        built.append(PackedAdapters(a_cat, b_cat, col_scale, spans))
    built[0].overflow = built[1:]
    return built[0]


def rescale_(packed: PackedAdapters, adapters: Dict[str, Adapter], global_scale: float = 1.0) -> None:
    """Rewrite col_scale only (scale_lora_layers / set_adapters weight change); A_cat/B_cat stay put."""
    for pk in [packed, *packed.overflow]:
        for n, c, r in pk.spans:
            pk.col_scale[c:c + r] = adapters[n].multiplier(global_scale)


# ---- per-block adapter scales -------------------------------------------------------------------------------------
# A per-adapter weight may be one number or a nested description of the UNet's transformers (the surface of
# diffusers-hf/src/diffusers/loaders/unet_loader_utils.py:41-141):
#     {"down": 2, "mid": 3, "up": {"block_0": 4, "block_1": [5, 6, 7]}}
# "mid" is one number; "down" / "up" are a number for the whole half, or a dict per block ("block_<i>") whose value is
# a number for the block or a list with one number per transformer of the block; whatever is left out counts as 1.
# The result maps the module path of every transformer ("up_blocks.1.attentions.2") to its number.

def _transformer_slots(blocks_with_transformer, transformer_per_block):
    """(user spelling, module path, half, block index, transformer index) of every Transformer2DModel, the order the
    reference's result dict has: mid, then up, then down."""
    slots = [("mid", "mid_block.attentions.0", "mid", None, None)]
    for half in ("up", "down"):
        for blk in blocks_with_transformer[half]:
            for j in range(transformer_per_block[half]):
                slots.append((f"{half}.block_{blk}.{j}", f"{half}_blocks.{blk}.attentions.{j}", half, blk, j))
    return slots


def _scale_of_slot(spec: dict, half: str, blk, j):
    node = spec.get(half, 1)
    if half == "mid":
        return node
    if isinstance(node, dict):
        node = node[f"block_{blk}"]      # a per-block dict must name every block that has transformers (KeyError)
    if isinstance(node, list):
        node = node[j]
    return node


def expand_lora_scales_for_one_adapter(scales, blocks_with_transformer: Dict[str, List[int]],
                                       transformer_per_block: Dict[str, int], module_names: Optional[Sequence[str]] = None):
    """Number in, number out; nested description in, {transformer module path: scale} out (see above).
    module_names: when given, every transformer path must occur inside at least one of them (the reference checks
    against the state-dict keys, unet_loader_utils.py:135-139), else ValueError."""
    for what, d in (("blocks_with_transformer", blocks_with_transformer), ("transformer_per_block", transformer_per_block)):
        if set(d) != {"down", "up"}:
            raise ValueError(f"{what} needs to be a dict with keys `'down' and `'up'`")
    if not isinstance(scales, dict):
        return scales
    out = {}
    for user_name, path, half, blk, j in _transformer_slots(blocks_with_transformer, transformer_per_block):
        if module_names is not None and not any(path in m for m in module_names):
            raise ValueError(f"Can't set lora scale for layer {user_name}. It either doesn't exist in this unet or "
                             "it has no attentions.")
        out[path] = _scale_of_slot(scales, half, blk, j)
    return out


def module_weight(weight_for_adapter, module_name: str) -> float:
    """The scale of one module: the float itself, or the first expanded layer name contained in the module's name
    (get_module_weight, diffusers-hf/src/diffusers/utils/peft_utils.py:241-249)."""
    if not isinstance(weight_for_adapter, dict):
        return float(weight_for_adapter)
    for layer_name, w in weight_for_adapter.items():
        if layer_name in module_name:
            return float(w)
    raise RuntimeError(f"No LoRA weight found for module {module_name}.")


def fold_layer_norm(weight: torch.Tensor, bias, gamma: torch.Tensor, beta, a_cat=None):
    """The operands of a linear whose LayerNorm (weight gamma, bias beta over the input features) is folded into the GEMM
    (kh_lora_linear_norm_bf16):  LN(x) W^T + b = rstd * (x W'^T - mean * c1) + c2.
    Returns (W', c1, c2, A', ca1, ca2): W' = W * gamma per input column (rounded to the weight's dtype), c1 the row sums
    of the rounded W', c2 = b + W beta; A' / ca1 / ca2 the same for the stacked adapter A matrices (None without)."""
    g = gamma.detach().double()
    b = None if beta is None else beta.detach().double()

    def terms(m):
        md = m.detach().double()
        mp = (md * g).to(m.dtype)
        s1 = mp.double().sum(dim=1)
        s2 = md @ b if b is not None else torch.zeros_like(s1)
        return mp.contiguous(), s1, s2

    wp, c1, c2 = terms(weight)
    if bias is not None:
        c2 = c2 + bias.detach().double()
    out = [wp, c1.float().contiguous(), c2.float().contiguous()]
    if a_cat is not None:
        ap, ca1, ca2 = terms(a_cat)
        out += [ap, ca1.float().contiguous(), ca2.float().contiguous()]
    else:
        out += [None, None, None]
    return tuple(out)
