"""HIP-graph capture of one UNet step.

The reference captures the step as two CUDA graphs (down+mid, then up) because remote ControlNet
residuals arrive between them (diffusers-hf/src/diffusers/models/unets/unet_2d_condition.py:1344-1526,
static inputs refreshed by recursive_copy :64-78).  On one GPU the residuals are ordinary inputs, so
one graph holds the whole step: ~1500 kernel launches replayed with a single hipGraphLaunch.
Every katz_hip op enqueues on torch's current stream and allocates nothing itself, so the capture
needs no special cases.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch


class GraphedUNetStep:
    """One captured step with static input / output tensors.

    The graph holds device addresses: of the weights, of the kernel-side weight copies (stacked q/k/v, interleaved
    GEGLU rows, packed convolution weights, stacked time_emb_proj), of the packed adapters and of the scratch buffers.
    It stays valid across everything that is written IN PLACE -- new inputs, adapter weights and the global LoRA scale
    (`set_adapters` with the same adapter set, `cross_attention_kwargs["scale"]`: only `col_scale` of the linear layers is
    rewritten; adapters on 3x3 convolutions repack on any change).
    After anything that repacks or re-derives buffers -- a different set of active adapters, `load_lora_into_unet` /
    `unload_lora`, `fuse_lora` / `unfuse_lora`, `patch_on_lora`, `load_state_dict`, another batch size or resolution --
    build a new GraphedUNetStep; replaying the old one would compute with the old buffers."""

    def __init__(self, unet, sample, timestep, encoder_hidden_states, added_cond_kwargs,
                 down_block_additional_residuals: Optional[Sequence[torch.Tensor]] = None,
                 mid_block_additional_residual: Optional[torch.Tensor] = None, warmup: int = 2):
        self.unet = unet
        cl = lambda t: t.detach().to(torch.bfloat16).contiguous(memory_format=torch.channels_last).clone()
        self.sample = cl(sample)
        self.timestep = torch.as_tensor(timestep, dtype=torch.float32, device=sample.device).reshape(-1).clone()
        self.ctx = encoder_hidden_states.detach().to(torch.bfloat16).contiguous().clone()
        self.added = {k: v.detach().clone() for k, v in added_cond_kwargs.items()}
        self.down = None if down_block_additional_residuals is None else [cl(r) for r in down_block_additional_residuals]
        self.mid = None if mid_block_additional_residual is None else cl(mid_block_additional_residual)
        unet.prepare()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side), torch.no_grad():
            for _ in range(warmup):   # workspace and counter allocation, lazy packing: all before capture
                self._run()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph), torch.no_grad():
            self.out = self._run()

    def _run(self):
        return self.unet(self.sample, self.timestep, self.ctx, added_cond_kwargs=self.added,
                         down_block_additional_residuals=self.down, mid_block_additional_residual=self.mid,
                         return_dict=False)[0]

    def __call__(self, sample=None, timestep=None, encoder_hidden_states=None, added_cond_kwargs=None,
                 down_block_additional_residuals=None, mid_block_additional_residual=None) -> torch.Tensor:
        """Refresh whichever static inputs are given, replay, return the (static) output tensor."""
        if sample is not None:
            self.sample.copy_(sample)
        if timestep is not None:
            self.timestep.copy_(torch.as_tensor(timestep, dtype=torch.float32).reshape(-1))
        if encoder_hidden_states is not None:
            self.ctx.copy_(encoder_hidden_states)
        if added_cond_kwargs is not None:
            for k, v in added_cond_kwargs.items():
                self.added[k].copy_(v)
        if down_block_additional_residuals is not None:
            for dst, src in zip(self.down, down_block_additional_residuals):
                dst.copy_(src)
        if mid_block_additional_residual is not None:
            self.mid.copy_(mid_block_additional_residual)
        self.graph.replay()
        return self.out

    def check(self) -> None:
        """Wait for the replays issued so far and raise ops.SplitTimeoutError if a bounded wait inside one of the
        step's LoRA launches ran out (the output of such a step is not trustworthy)."""
        from . import ops

        ops.check_split_timeouts(self.sample.device)
