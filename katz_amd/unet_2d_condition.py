"""UNet2DConditionModel (SDXL configuration) on the katz_hip kernels.

Drop-in for the reference's model at the call boundary
(diffusers-hf/src/diffusers/models/unets/unet_2d_condition.py:1955-1974): same forward keyword
arguments -- including ControlNet's `down_block_additional_residuals` / `mid_block_additional_residual`
and the Katz extras `controlnet_skt, serve_mode, time_stats, controlnet_num` -- same module / state-dict
names, and the LoRA surface (`load_lora_into_unet`, `set_adapters`, `fuse_lora`, `unfuse_lora`,
`unload_lora`, `disable_lora` / `enable_lora`, `cross_attention_kwargs={"scale": s}`) of
diffusers-hf/src/diffusers/loaders/unet.py:514-618 and diffusers-hf/src/diffusers/loaders/lora.py:382-496,
implemented without peft: every LoRA-able Linear is a `LoRALinear` that runs the fused kernel.

Semantics follow the reference's CUDA-graph path (_down_forward :1127-1252, _up_forward :1254-1341),
which adds all nine skip residuals and the mid residual; the eager variant's `is not None` guard that
drops the skip adds (:1886-1898) is not reproduced.
"""
from __future__ import annotations

import math
import re
from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Sequence, Tuple, Union

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops
from .layers import Conv3x3, LoRALinear, TimestepEmbedding, fused_norm_silu
from .lora import expand_lora_scales_for_one_adapter, module_weight
from .unet_blocks import (CrossAttnDownBlock2D, CrossAttnUpBlock2D, DownBlock2D, UNetMidBlock2DCrossAttn, UpBlock2D)


@dataclass
class UNetConfig:
    in_channels: int = 4
    out_channels: int = 4
    block_out_channels: Tuple[int, ...] = (320, 640, 1280)
    down_block_types: Tuple[str, ...] = ("DownBlock2D", "CrossAttnDownBlock2D", "CrossAttnDownBlock2D")
    up_block_types: Tuple[str, ...] = ("CrossAttnUpBlock2D", "CrossAttnUpBlock2D", "UpBlock2D")
    layers_per_block: int = 2
    transformer_layers_per_block: Tuple[int, ...] = (1, 2, 10)
    num_attention_heads: Tuple[int, ...] = (5, 10, 20)  # stored as `attention_head_dim` in SDXL's config.json
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
        return UNetConfig(block_out_channels=(64, 128, 256), transformer_layers_per_block=(1, 1, 2),
                          num_attention_heads=(1, 2, 4), cross_attention_dim=128, addition_time_embed_dim=32,
                          projection_class_embeddings_input_dim=64 + 6 * 32)


@dataclass
class UNet2DConditionOutput:
    sample: torch.Tensor


_freq_tables: Dict[tuple, torch.Tensor] = {}


def _frequencies(half: int, downscale_freq_shift: float, max_period: int, device) -> torch.Tensor:
    """exp(-ln(max_period) * arange(half) / (half - shift)) (embeddings.py:50-55): constants of the model, computed
    once per device with the reference's own sequence of operations instead of in every step."""
    key = (half, float(downscale_freq_shift), int(max_period), device.type, device.index)
    t = _freq_tables.get(key)
    if t is None:
        exponent = -math.log(max_period) * torch.arange(0, half, dtype=torch.float32, device=device)
        t = torch.exp(exponent / (half - downscale_freq_shift))
        if not (device.type == "cuda" and torch.cuda.is_current_stream_capturing()):
            _freq_tables[key] = t   # a tensor made during graph capture lives in the graph's pool: do not keep it
    return t


def get_timestep_embedding(timesteps, embedding_dim, flip_sin_to_cos=False, downscale_freq_shift=1.0, scale=1.0,
                           max_period=10000):
    """diffusers-hf/src/diffusers/models/embeddings.py:26-66, evaluated on the device of `timesteps`."""
    half = embedding_dim // 2
    emb = scale * timesteps[:, None].float() * _frequencies(half, downscale_freq_shift, max_period, timesteps.device)[None, :]
    emb = torch.cat([torch.sin(emb), torch.cos(emb)], dim=-1)
    if flip_sin_to_cos:
        emb = torch.cat([emb[:, half:], emb[:, :half]], dim=-1)
    if embedding_dim % 2 == 1:
        emb = F.pad(emb, (0, 1, 0, 0))
    return emb


# LoRA key spellings accepted by load_lora_into_unet -> (module path, "down" | "up")
_LORA_PATTERNS = [
    (re.compile(r"^(.*)\.processor\.(to_q|to_k|to_v|to_out)_lora\.(down|up)\.weight$"), "processor"),
    (re.compile(r"^(.*)\.(to_q|to_k|to_v)_lora\.(down|up)\.weight$"), "attn_old"),
    (re.compile(r"^(.*)\.lora\.(down|up)\.weight$"), "plain"),
    (re.compile(r"^(.*)\.lora_(A|B)(?:\.[^.]+)?\.weight$"), "peft"),
]


def parse_lora_key(key: str) -> Optional[Tuple[str, str]]:
    """Map one LoRA state-dict key to (UNet module path, 'down'|'up').

    Spellings: the kohya->diffusers converted keys the reference stores in shared memory
    (`<attn>.processor.to_q_lora.down.weight`, `<module>.lora.up.weight`; lora_info_shm/*_key_match_unet.json,
    built by gen_lora_diffuser_key_match.py:131-175) and the peft spelling they are converted to
    (`<module>.lora_A.weight`, diffusers-hf/src/diffusers/utils/state_dict_utils.py:38-50)."""
    if key.startswith("unet."):
        key = key[len("unet."):]
    for pat, kind in _LORA_PATTERNS:
        m = pat.match(key)
        if not m:
            continue
        if kind == "processor" or kind == "attn_old":
            proj = m.group(2)
            mod = f"{m.group(1)}.{'to_out.0' if proj == 'to_out' else proj}"
            return mod, m.group(3)
        if kind == "plain":
            return m.group(1), m.group(2)
        return m.group(1), "down" if m.group(2) == "A" else "up"
    return None


class UNet2DConditionModel(nn.Module):
    def __init__(self, cfg: Optional[UNetConfig] = None):
        super().__init__()
        cfg = cfg or UNetConfig.sdxl()
        self.cfg = cfg
        boc = cfg.block_out_channels
        ted = boc[0] * 4
        self.conv_in = Conv3x3(cfg.in_channels, boc[0])
        self.time_embedding = TimestepEmbedding(boc[0], ted)
        self.add_embedding = TimestepEmbedding(cfg.projection_class_embeddings_input_dim, ted)
        n = len(boc)
        self.down_blocks = nn.ModuleList()
        out_ch = boc[0]
        for i, typ in enumerate(cfg.down_block_types):
            in_ch, out_ch = out_ch, boc[i]
            common = dict(in_channels=in_ch, out_channels=out_ch, temb_channels=ted, num_layers=cfg.layers_per_block,
                          resnet_eps=cfg.norm_eps, resnet_groups=cfg.norm_num_groups, add_downsample=i != n - 1)
            if typ == "DownBlock2D":
                self.down_blocks.append(DownBlock2D(**common))
            elif typ == "CrossAttnDownBlock2D":
                self.down_blocks.append(CrossAttnDownBlock2D(
                    **common, transformer_layers_per_block=cfg.transformer_layers_per_block[i],
                    num_attention_heads=cfg.num_attention_heads[i], cross_attention_dim=cfg.cross_attention_dim,
                    use_linear_projection=cfg.use_linear_projection))
            else:
                raise ValueError(f"unsupported down block {typ}")
        self.mid_block = UNetMidBlock2DCrossAttn(
            in_channels=boc[-1], temb_channels=ted, transformer_layers_per_block=cfg.transformer_layers_per_block[-1],
            resnet_eps=cfg.norm_eps, resnet_groups=cfg.norm_num_groups, num_attention_heads=cfg.num_attention_heads[-1],
            cross_attention_dim=cfg.cross_attention_dim, use_linear_projection=cfg.use_linear_projection)
        self.up_blocks = nn.ModuleList()
        rev, rev_heads = list(reversed(boc)), list(reversed(cfg.num_attention_heads))
        rev_tl = list(reversed(cfg.transformer_layers_per_block))
        out_ch = rev[0]
        for i, typ in enumerate(cfg.up_block_types):
            prev, out_ch = out_ch, rev[i]
            in_ch = rev[min(i + 1, n - 1)]
            common = dict(in_channels=in_ch, out_channels=out_ch, prev_output_channel=prev, temb_channels=ted,
                          num_layers=cfg.layers_per_block + 1, resnet_eps=cfg.norm_eps,
                          resnet_groups=cfg.norm_num_groups, add_upsample=i != n - 1)
            if typ == "UpBlock2D":
                self.up_blocks.append(UpBlock2D(**common))
            elif typ == "CrossAttnUpBlock2D":
                self.up_blocks.append(CrossAttnUpBlock2D(
                    **common, transformer_layers_per_block=rev_tl[i], num_attention_heads=rev_heads[i],
                    cross_attention_dim=cfg.cross_attention_dim, use_linear_projection=cfg.use_linear_projection))
            else:
                raise ValueError(f"unsupported up block {typ}")
        self.conv_norm_silu = nn.Sequential(*fused_norm_silu(boc[0], cfg.norm_num_groups, cfg.norm_eps))
        self.conv_out = Conv3x3(boc[0], cfg.out_channels)
        self.num_upsamplers = n - 1
        self._ctx_kv = None
        # The reference's switches (read at construction, unet_2d_condition.py:511, resnet.py:330, normalization.py:31).
        # ENABLE_CUDA_GRAPH=1: forward replays a captured HIP graph of the step (see _forward_graphed).
        # ENABLE_FUSED_NORM_SILU / ENABLE_CHANNELS_LAST: accepted and recorded; this build always runs the fused
        # GroupNorm+SiLU kernel on NHWC memory, which is what the reference does with both switched on, so they change
        # nothing here.  ENABLE_FUSED_GEGLU is read by layers.GEGLU.
        from .layers import env_flag
        self.enable_cuda_graph = env_flag("ENABLE_CUDA_GRAPH")
        self.enable_fused_norm_silu = env_flag("ENABLE_FUSED_NORM_SILU")
        self.enable_channels_last = env_flag("ENABLE_CHANNELS_LAST")
        self._graphs: Dict[tuple, Any] = {}
        self._register_load_state_dict_pre_hook(self._remap_upstream_keys)

    # ---- checkpoints ---------------------------------------------------------------------------
    @staticmethod
    def _remap_upstream_keys(state_dict, prefix, *args):
        """Accept upstream-diffusers key names, as the reference's load hooks do:
        conv_norm_out.* -> conv_norm_silu.0.* (unet_2d_condition.py:521-529),
        resnet norm1/norm2 -> norm_silu1.0/norm_silu2.0 (diffusers-hf/src/diffusers/models/resnet.py:336-350),
        and the fused-GEGLU split proj_1 / proj_2 -> proj (activations.py:151-170, inverted)."""
        for k in list(state_dict.keys()):
            nk = k
            if k.startswith(prefix + "conv_norm_out."):
                nk = k.replace("conv_norm_out.", "conv_norm_silu.0.", 1)
            elif re.search(r"\.resnets\.\d+\.norm[12]\.(weight|bias)$", k):
                nk = re.sub(r"\.norm([12])\.(weight|bias)$", r".norm_silu\1.0.\2", k)
            if nk != k:
                state_dict[nk] = state_dict.pop(k)
        for k in [k for k in state_dict if ".ff.net.0.proj_1." in k]:
            k2 = k.replace(".proj_1.", ".proj_2.")
            if k2 in state_dict:  # proj_1 = value half, proj_2 = gate half of `proj` (chunk(2, dim=0))
                state_dict[k.replace(".proj_1.", ".proj.")] = torch.cat([state_dict.pop(k), state_dict.pop(k2)], dim=0)

    def to_runtime(self, device="cuda", dtype=torch.bfloat16) -> "UNet2DConditionModel":
        """Move to the GPU in the kernel formats: bf16, conv weights channels_last, packed GEGLU rows."""
        self.to(device=device, dtype=dtype)
        self.to(memory_format=torch.channels_last)
        self.prepare()
        return self.eval()

    def prepare(self) -> None:
        for m in self.lora_linears().values():
            m.prepare()
        if self._ctx_kv is None:
            from .layers import Attention, ContextKVProjector, ResnetBlock2D, TimeEmbProjector
            self._ctx_kv = ContextKVProjector([m for m in self.modules() if isinstance(m, Attention)])
            self._temb_proj = TimeEmbProjector([m for m in self.modules() if isinstance(m, ResnetBlock2D)])

    # ---- LoRA surface ----------------------------------------------------------------------------
    def lora_linears(self) -> Dict[str, LoRALinear]:
        return {n: m for n, m in self.named_modules() if isinstance(m, LoRALinear)}

    def lora_convs(self) -> Dict[str, Any]:
        """Convolutions that can carry a LoRA: 3x3 (resnet conv1 / conv2, down / upsampler convs) and the resnets' 1x1
        conv_shortcut."""
        from .layers import Conv1x1, Conv3x3
        return {n: m for n, m in self.named_modules() if isinstance(m, (Conv3x3, Conv1x1))}

    def _lora_targets(self) -> Dict[str, Any]:
        return {**self.lora_linears(), **self.lora_convs()}

    def load_lora_into_unet(self, state_dict: Dict[str, torch.Tensor], network_alphas: Optional[Dict[str, float]] = None,
                            adapter_name: Optional[str] = None) -> str:
        """Register one adapter from a LoRA state dict (load_lora_into_unet,
        diffusers-hf/src/diffusers/loaders/lora.py:382-496).  Keys in any spelling parse_lora_key accepts;
        keys of other components (text encoders) are ignored; network_alphas maps
        "<module or down key>.alpha" to alpha (:261-270), default alpha = rank."""
        lin = self._lora_targets()
        pairs: Dict[str, Dict[str, torch.Tensor]] = {}
        for k, v in state_dict.items():
            if k.startswith("text_encoder"):
                continue
            parsed = parse_lora_key(k)
            if parsed is None:
                continue
            mod, which = parsed
            pairs.setdefault(mod, {})[which] = v
            pairs[mod][which + "_key"] = k
        if not pairs:
            raise ValueError("no UNet LoRA keys found in the state dict")
        adapter_name = adapter_name or f"default_{len(self.adapter_names())}"
        if adapter_name in self.adapter_names():
            raise ValueError(f"adapter name {adapter_name!r} is already in use in the UNet")
        for mod, pr in pairs.items():
            if mod not in lin:
                raise ValueError(f"LoRA targets {mod!r}, which is not a LoRA-able linear or 3x3 convolution of this UNet")
            if "down" not in pr or "up" not in pr:
                raise ValueError(f"LoRA for {mod!r} lacks its {'down' if 'down' not in pr else 'up'} matrix")
            alpha = None
            if network_alphas:
                for cand in (pr["down_key"] + ".alpha", "unet." + mod + ".alpha", mod + ".alpha",
                             pr["down_key"].removeprefix("unet.") + ".alpha"):
                    if cand in network_alphas:
                        alpha = float(network_alphas[cand])
                        break
            lin[mod].add_adapter(adapter_name, pr["down"], pr["up"], alpha)
        self.set_adapters(self.adapter_names())  # a freshly loaded adapter is active, like peft's
        return adapter_name

    def adapter_names(self) -> List[str]:
        names: List[str] = []
        for m in self._lora_targets().values():
            for n in m.adapters:
                if n not in names:
                    names.append(n)
        return names

    def set_adapters(self, adapter_names: Union[str, Sequence[str]],
                     weights: Optional[Union[float, Sequence[float]]] = None) -> None:
        """UNet2DConditionLoadersMixin.set_adapters, diffusers-hf/src/diffusers/loaders/unet.py:565-618."""
        names = [adapter_names] if isinstance(adapter_names, str) else list(adapter_names)
        if weights is None:
            weights = [1.0] * len(names)
        elif isinstance(weights, (int, float, dict)):
            weights = [weights] * len(names)
        if len(weights) != len(names):
            raise ValueError(f"Length of adapter names {len(names)} is not equal to the length of their weights {len(weights)}.")
        weights = [1.0 if w is None else w for w in weights]
        lin = self._lora_targets()
        if any(isinstance(w, dict) for w in weights):
            # per-block scales, e.g. {"down": 0.9, "mid": 1.0, "up": {"block_0": 0.6, "block_1": [0.4, 0.8, 1.0]}}
            # (_maybe_expand_lora_scales, diffusers-hf/src/diffusers/loaders/unet_loader_utils.py:41-58)
            bwt = {"down": [i for i, b in enumerate(self.down_blocks) if hasattr(b, "attentions")],
                   "up": [i for i, b in enumerate(self.up_blocks) if hasattr(b, "attentions")]}
            tpb = {"down": self.cfg.layers_per_block, "up": self.cfg.layers_per_block + 1}
            weights = [expand_lora_scales_for_one_adapter(w, bwt, tpb, list(lin.keys())) for w in weights]
        for mod_name, m in lin.items():
            # per-block dictionaries address transformers only; other modules (resnet convs) keep scale 1 under them
            m.set_active(names, [module_weight(w, mod_name) if (not isinstance(w, dict) or ".attentions." in mod_name) else 1.0
                                 for w in weights])

    def disable_lora(self) -> None:
        for m in self._lora_targets().values():
            m.adapters_enabled = False
            m.refresh_adapters()

    def enable_lora(self) -> None:
        for m in self._lora_targets().values():
            m.adapters_enabled = True
            m.refresh_adapters()

    def fuse_lora(self, lora_scale: float = 1.0, adapter_names: Optional[Sequence[str]] = None,
                  safe_fusing: bool = False) -> None:
        """W += lora_scale * weight_i * alpha_i / rank_i * B_i A_i for the named (default: active) adapters of every
        target (fuse_lora, diffusers-hf/src/diffusers/loaders/unet.py:514-550 -> _fuse_lora, models/lora.py:403-433,
        :258-296 for convolutions).  safe_fusing=False (the reference's default): all linear layers in one launch per
        adapter of the batched merge kernel.  safe_fusing=True: layer by layer in fp32 with the reference's finite
        check (:416-421), all layers or none -- a layer that fails raises and the layers merged before it get their
        weights back bit for bit."""
        if not safe_fusing and self._merge_grouped(lora_scale, adapter_names):
            for c in self.lora_convs().values():
                c.fuse(lora_scale, adapter_names)
            return
        done = []
        try:
            for m in self._lora_targets().values():
                names = list(m.active if adapter_names is None else adapter_names)
                cand = m._fuse_candidate(lora_scale, names)
                if cand is not None:
                    done.append((m, m.weight.detach().clone(), dict(m._fused)))
                    m._fuse_commit(*cand)
        except Exception:
            with torch.no_grad():
                for m, w0, fused0 in reversed(done):
                    m.weight.copy_(w0)
                    m._fused = fused0
                    m.refresh_adapters()
            raise

    def _merge_grouped(self, lora_scale: float, adapter_names: Optional[Sequence[str]], undo: bool = False) -> bool:
        """Fuse (or, with undo, unfuse) the adapters of all LoRALinear layers with the batched merge kernel; False when
        the weights are not bf16 on a GPU (the caller then takes the per-layer path)."""
        lin = list(self.lora_linears().values())
        if not lin or any((not m.weight.is_cuda) or m.weight.dtype != torch.bfloat16 for m in lin):
            return False
        rounds: List[List[tuple]] = []      # round k: the k-th adapter to merge of every layer (a weight once per launch)
        for m in lin:
            if undo:
                todo = list(m._fused.items())
            else:
                names = list(m.active if adapter_names is None else adapter_names)
                todo, seen = [], set()
                for n in names:
                    if n in m.adapters and n not in m._fused and n not in seen:
                        todo.append((n, lora_scale * m.adapters[n].multiplier(1.0)))
                        seen.add(n)
            for k, (n, mult) in enumerate(todo):
                if len(rounds) <= k:
                    rounds.append([])
                rounds[k].append((m, n, mult))
        dev = lin[0].weight.device
        with torch.no_grad():
            for rnd in rounds:
                ops.lora_merge_grouped([m.weight.data for m, _, _ in rnd],
                                       [m.adapters[n].up.to(dev, torch.bfloat16).contiguous() for m, n, _ in rnd],
                                       [m.adapters[n].down.to(dev, torch.bfloat16).contiguous() for m, n, _ in rnd],
                                       scale=-1.0 if undo else 1.0, layer_scales=[mult for _, _, mult in rnd])
        for m in lin:
            torch.autograd.graph.increment_version(m.weight)
        for rnd in rounds:
            for m, n, mult in rnd:
                if undo:
                    m._fused.pop(n, None)
                else:
                    m._fused[n] = mult
        for m in lin:
            m.refresh_adapters()
        return True

    def unfuse_lora(self) -> None:
        if self._merge_grouped(1.0, None, undo=True):
            for c in self.lora_convs().values():
                c.unfuse()
            return
        for m in self._lora_targets().values():
            m.unfuse()

    def unload_lora(self) -> None:
        for m in self.lora_linears().values():
            if m._fused:
                m.unfuse()
            for n in list(m.adapters):
                m.delete_adapter(n)
            m.refresh_adapters()
        for c in self.lora_convs().values():
            if c._fused:
                c.unfuse()
            for n in list(c.adapters):
                c.delete_adapter(n)

    def delete_adapters(self, adapter_names: Union[str, Sequence[str]]) -> None:
        names = [adapter_names] if isinstance(adapter_names, str) else list(adapter_names)
        for m in self._lora_targets().values():
            for n in names:
                m.delete_adapter(n)
            m.refresh_adapters()

    def scale_lora_layers(self, scale: float) -> None:
        for m in self._lora_targets().values():
            m.set_global_scale(scale)

    def set_attn_processor(self, processor) -> None:
        """unet_2d_condition.py:800-832: one processor for all, or a dict keyed '<module>.processor'."""
        from .layers import Attention
        for name, m in self.named_modules():
            if isinstance(m, Attention):
                m.set_processor(processor[f"{name}.processor"] if isinstance(processor, dict) else processor)

    @property
    def attn_processors(self) -> Dict[str, Any]:
        from .layers import Attention
        return {f"{n}.processor": m.get_processor() for n, m in self.named_modules() if isinstance(m, Attention)}

    # ---- forward -------------------------------------------------------------------------------------
    def _embed(self, sample, timestep, added_cond_kwargs):
        cfg = self.cfg
        B = sample.shape[0]
        if not torch.is_tensor(timestep):
            timestep = torch.tensor([timestep], dtype=torch.float32, device=sample.device)
        t = timestep.reshape(-1).to(sample.device)
        if t.numel() == 1:
            t = t.expand(B)
        t_emb = get_timestep_embedding(t, cfg.block_out_channels[0], flip_sin_to_cos=True, downscale_freq_shift=0)
        emb = self.time_embedding(t_emb.to(sample.dtype))
        if added_cond_kwargs is None or "text_embeds" not in added_cond_kwargs or "time_ids" not in added_cond_kwargs:
            raise ValueError("addition_embed_type 'text_time' requires `text_embeds` and `time_ids` in `added_cond_kwargs`")
        text_embeds, time_ids = added_cond_kwargs["text_embeds"], added_cond_kwargs["time_ids"]
        tid = get_timestep_embedding(time_ids.flatten(), cfg.addition_time_embed_dim, flip_sin_to_cos=True,
                                     downscale_freq_shift=0).reshape(B, -1)
        add = torch.cat([text_embeds.to(sample.dtype), tid.to(sample.dtype)], dim=-1)
        return emb + self.add_embedding(add)

    @staticmethod
    def _residual_sets(res, n_expected):
        """Normalise ControlNet residuals to a list (per skip) of lists (per ControlNet) of channels_last tensors."""
        if res is None:
            return [[] for _ in range(n_expected)]
        res = list(res)
        if len(res) and isinstance(res[0], (list, tuple)):   # several ControlNets: list of residual sets
            sets = [list(s) for s in res]
            if any(len(s) != n_expected for s in sets):
                raise ValueError(f"every ControlNet residual set must hold {n_expected} tensors")
            per_skip = [[s[j] for s in sets] for j in range(n_expected)]
        else:
            if len(res) != n_expected:
                raise ValueError(f"expected {n_expected} down-block residuals, got {len(res)}")
            per_skip = [[r] for r in res]
        return [[r.to(torch.bfloat16).contiguous(memory_format=torch.channels_last) for r in rs] for rs in per_skip]

    def _forward_graphed(self, sample, timestep, ctx, cross_attention_kwargs, added, down, mid):
        """ENABLE_CUDA_GRAPH=1: the step as a captured graph, built on the first call with a given signature (input
        shapes, which residuals are given, the packed-adapter generation, the global LoRA scale) and replayed with
        refreshed static inputs afterwards -- what _forward_w_separate_cuda_graph does with its two graphs
        (unet_2d_condition.py:1344-1526, static inputs refreshed by recursive_copy :64-78).  The returned tensor is
        the graph's static output: it is overwritten by the next call with the same signature."""
        from . import layers as L
        from .graph import GraphedUNetStep

        scale = 1.0 if cross_attention_kwargs is None else float(cross_attention_kwargs.get("scale", 1.0))
        self.scale_lora_layers(scale)
        multi = bool(down) and isinstance(down[0], (list, tuple))
        if multi or isinstance(mid, (list, tuple)):
            raise NotImplementedError("ENABLE_CUDA_GRAPH=1 takes one ControlNet residual set; average several first")
        key = (tuple(sample.shape), tuple(ctx.shape), None if down is None else len(down), mid is not None,
               L._pack_epoch, scale, tuple(sorted((k, tuple(v.shape)) for k, v in added.items())))
        g = self._graphs.get(key)
        if g is None:
            if len(self._graphs) >= 4:      # adapters changed or a new resolution: old graphs hold dead buffers
                self._graphs.clear()
            self._building_graph = True
            try:
                with torch.no_grad():
                    g = GraphedUNetStep(self, sample, timestep, ctx, added, down, mid)
            finally:
                self._building_graph = False
            self._graphs[key] = g
        out = g(sample, timestep, ctx, added, down, mid)
        if cross_attention_kwargs is not None:
            self.scale_lora_layers(1.0)
        return out

    def forward(self, sample, timestep, encoder_hidden_states, class_labels=None, timestep_cond=None,
                attention_mask=None, cross_attention_kwargs=None, added_cond_kwargs=None,
                down_block_additional_residuals=None, mid_block_additional_residual=None,
                down_intrablock_additional_residuals=None, encoder_attention_mask=None, return_dict: bool = True,
                controlnet_skt=None, serve_mode=None, time_stats=None, controlnet_num=None):
        if (self.enable_cuda_graph and sample.is_cuda and not torch.cuda.is_current_stream_capturing()
                and not getattr(self, "_building_graph", False)):
            out = self._forward_graphed(sample, timestep, encoder_hidden_states, cross_attention_kwargs,
                                        added_cond_kwargs, down_block_additional_residuals,
                                        mid_block_additional_residual)
            return (out,) if not return_dict else UNet2DConditionOutput(sample=out)
        for name, val in (("class_labels", class_labels), ("timestep_cond", timestep_cond),
                          ("attention_mask", attention_mask), ("encoder_attention_mask", encoder_attention_mask),
                          ("down_intrablock_additional_residuals", down_intrablock_additional_residuals),
                          ("controlnet_skt", controlnet_skt)):
            if val is not None:
                raise NotImplementedError(f"`{name}` is not used on the SDXL + ControlNet + LoRA path and is not implemented")
        if cross_attention_kwargs is not None:
            self.scale_lora_layers(float(cross_attention_kwargs.get("scale", 1.0)))
        if sample.dtype != torch.bfloat16 or not sample.is_contiguous(memory_format=torch.channels_last):
            sample = sample.to(torch.bfloat16).contiguous(memory_format=torch.channels_last)
        ctx = encoder_hidden_states.to(torch.bfloat16).contiguous()
        if sample.is_cuda:
            ops.split_counters_reset(sample.device)   # one fill per step clears the in-launch shrinks' counters

        with ops.weight_prefetch_scope(self):   # hints are learned from, and point into, this model's own last pass
            if self._ctx_kv is None:
                self.prepare()
            if not getattr(self, "context_kv_ready", False):   # (a denoise loop projects its one text context once, not per step)
                self._ctx_kv.run(ctx)  # K/V projections of all cross-attentions, grouped
            emb = self._embed(sample, timestep, added_cond_kwargs)
            temb_act = F.silu(emb)
            self._temb_proj.run(temb_act)   # time_emb_proj of all resnets, batched per width
            sample = self.conv_in(sample)
            skips = (sample,)
            for blk in self.down_blocks:
                sample, res = blk(sample, temb_act, ctx)
                skips += res
            sample = self.mid_block(sample, temb_act, ctx)

            ready = getattr(self, "before_residuals", None)
            if ready is not None:   # the residuals come from another stream (a ControlNet run beside the down blocks)
                ready()
            extra = self._residual_sets(down_block_additional_residuals, len(skips))
            if mid_block_additional_residual is not None:
                mids = mid_block_additional_residual
                mids = list(mids) if isinstance(mids, (list, tuple)) else [mids]
                mids = [m.to(torch.bfloat16).contiguous(memory_format=torch.channels_last) for m in mids]
                if not sample.is_contiguous(memory_format=torch.channels_last):
                    sample = sample.contiguous(memory_format=torch.channels_last)
                sample = ops.residual_add_(sample, mids)

            for blk in self.up_blocks:
                n = len(blk.resnets)
                res, skips = skips[-n:], skips[:-n]
                ex, extra = extra[-n:], extra[:-n]
                sample = blk(sample, res, ex, temb_act, ctx)
            sample = self.conv_norm_silu(sample)
            if not getattr(self, "defer_conv_out", False):   # the denoise-loop graph runs conv_out fused with the scheduler step
                sample = self.conv_out(sample)
        if cross_attention_kwargs is not None:
            self.scale_lora_layers(1.0)  # unscale_lora_layers, unet_2d_condition.py:1334-1336
        if not return_dict:
            return (sample,)
        return UNet2DConditionOutput(sample=sample)
