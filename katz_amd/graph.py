"""HIP-graph capture of one UNet step.

The reference captures the step as two CUDA graphs (down+mid, then up) because remote ControlNet
residuals arrive between them (diffusers-hf/src/diffusers/models/unets/unet_2d_condition.py:1344-1526,
static inputs refreshed by recursive_copy :64-78).  On one GPU the residuals are ordinary inputs, so
one graph holds the whole step: ~1500 kernel launches replayed with a single hipGraphLaunch.
Every katz_hip op enqueues on torch's current stream and allocates nothing itself, so the capture
needs no special cases.
"""
from __future__ import annotations

import os
from typing import Dict, List, Optional, Sequence

import torch


class GraphedUNetStep:
    """One captured step with static input / output tensors.

    The graph holds device addresses: of the weights, of the kernel-side weight copies (stacked q/k/v, interleaved
    GEGLU rows, the copies scaled by a folded LayerNorm's weight, packed convolution weights, stacked time_emb_proj), of
    the packed adapters and of the scratch buffers.
    It stays valid across everything that is written IN PLACE -- new inputs, adapter weights and the global LoRA scale
    (`set_adapters` with the same adapter set, `cross_attention_kwargs["scale"]`: only `col_scale` of the linear layers is
    rewritten; adapters on 3x3 convolutions repack on any change).
    After anything that repacks or re-derives buffers -- a different set of active adapters, `load_lora_into_unet` /
    `unload_lora`, `fuse_lora` / `unfuse_lora`, `patch_on_lora`, `load_state_dict`, another batch size or resolution --
    build a new GraphedUNetStep; replaying the old one would compute with the old buffers.
    Weight-prefetch hints recorded in the graph point at tensors of this UNet only (they are learned and issued inside
    one forward of one model, ops.weight_prefetch_scope), so freeing ANOTHER model never invalidates this graph."""

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


class GraphedDenoiseStep:
    """One step of the guided ControlNet loop -- ControlNet -> UNet with its residuals -> guidance + Euler update + the
    next step's scaled, duplicated input -- as ONE captured graph (the body of the reference's loop,
    diffusers-hf/src/diffusers/pipelines/controlnet/pipeline_controlnet_sd_xl_katz.py:1509-1675; the reference splits
    it over processes and two graphs per UNet because its ControlNets run elsewhere, unet_2d_condition.py:1344-1526).

    Static state: the latents [B,4,H,W], the model input [2B,4,H,W] (both updated in place by the last kernel of the
    graph) and one fp32 row {sigma_i, sigma_{i+1}, sqrt(sigma_{i+1}^2 + 1), sqrt(sigma_i^2 + 1), timestep_i} that
    `run` rewrites before every replay; so one graph serves all steps of a schedule.

    The UNet's conv_out does not run as a convolution of its own: the graph ends with kh_conv_out_cfg_euler_bf16, which
    computes it and applies guidance, the Euler update and the next input's scaling in its epilogue (fuse_tail=False
    keeps conv_out and the scheduler kernel apart, as the eager denoise_loop runs them).

    overlap (default on, KATZ_CN_OVERLAP=0 switches it off): inside the graph the ControlNet runs on a second stream
    beside the UNet's down and mid blocks, which do not read its residuals; the UNet waits for it right after its mid
    block.  Same kernels, same results bit for bit; the 50-step loop at 1024x1024 measured 1769 -> 1610 ms.

    Build it (and call `run`) from a stream that is neither capturing nor itself a fork inside someone else's capture:
    with overlap on, the capture forks a second stream from the capturing one, and a fork from an already forked stream
    inside a capture has crashed the runtime at capture end; the constructor refuses to start under a capture.

    hoist_context_kv (default on): the to_k / to_v projections of all cross-attentions (with their adapters) read the text
    context only, which does not change during a loop; they run once per `run` (for both models) instead of in every step
    (the reference projects the context again in every step, attention_processor.py:1246-1251; same values, bit for bit:
    the same kernels on the same inputs).  The graph then reads their result buffers, so a change of the adapters' scales
    takes effect for these layers at the next `run`.

    hoist_cond_embedding: the ControlNet's conditioning embedding depends on the image only, which is the same in every
    step; it is computed once per `run` instead of inside the graph (the reference recomputes it every step,
    controlnet.py:780-783; same value, bit for bit).  Everything the notes on GraphedUNetStep say about rebuilding after
    adapters are repacked applies here too."""

    def __init__(self, unet, controlnet, latents, encoder_hidden_states, added_cond_kwargs, controlnet_cond,
                 guidance_scale: float, conditioning_scale: float = 0.5, hoist_cond_embedding: bool = True,
                 warmup: int = 2, fuse_tail: bool = True, overlap: Optional[bool] = None, hoist_context_kv: bool = True):
        from . import ops

        if latents.is_cuda and torch.cuda.is_current_stream_capturing():
            raise RuntimeError("GraphedDenoiseStep captures a graph of its own (with a forked stream when overlap is on): "
                               "build it outside any stream capture")
        self.unet, self.controlnet = unet, controlnet
        self.overlap = (os.getenv("KATZ_CN_OVERLAP", "1") != "0") if overlap is None else bool(overlap)
        self._cn_stream = torch.cuda.Stream(device=latents.device) if self.overlap else None
        self.guidance_scale, self.conditioning_scale = float(guidance_scale), float(conditioning_scale)
        dev = latents.device
        bf = torch.bfloat16
        cl = lambda t: t.detach().to(bf).contiguous(memory_format=torch.channels_last).clone()
        self.latents = cl(latents)
        self.model_input = cl(torch.cat([latents] * 2))
        self.ctx = encoder_hidden_states.detach().to(bf).contiguous().clone()
        self.added = {k: v.detach().clone() for k, v in added_cond_kwargs.items()}
        self.cond = cl(controlnet_cond)
        self.row = torch.zeros(5, dtype=torch.float32, device=dev)
        self.row[:4] = torch.tensor([1.0, 0.5, 1.0, 1.0])     # harmless values for the warm-up runs
        self.row[4] = 500.0
        self.hoist = hoist_cond_embedding
        self.hoist_kv = bool(hoist_context_kv)
        self.cond_emb = None
        co = unet.conv_out
        self.fuse_tail = bool(fuse_tail and co.in_channels % 16 == 0 and co.out_channels == 4 and not co.adapters)
        self._co_w = ops.pack_conv3x3_weight(co.weight) if self.fuse_tail else None   # [4,3,3,C], packed once
        unet.prepare()
        controlnet.prepare()
        keep = (self.latents.clone(), self.model_input.clone())
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side), torch.no_grad():
            if self.hoist:
                self.cond_emb = controlnet.embed_condition(self.cond)
            self._project_context()
            for _ in range(warmup):
                self._step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.latents.copy_(keep[0]); self.model_input.copy_(keep[1])
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph), torch.no_grad():
            self._step()
        self.latents.copy_(keep[0]); self.model_input.copy_(keep[1])
        self._ops = ops

    def _project_context(self):
        """The context K / V of both models from the static context tensor (hoist_context_kv)."""
        if self.hoist_kv:
            for m in (self.controlnet, self.unet):
                m._ctx_kv.run(self.ctx)

    def _step(self):
        from . import ops

        t = self.row[4:5]
        self.unet.context_kv_ready = self.controlnet.context_kv_ready = self.hoist_kv
        try:
            self._step_models(t)
        finally:
            self.unet.context_kv_ready = self.controlnet.context_kv_ready = False

    def _step_models(self, t):
        from . import ops

        if self.overlap:
            eps = self._models_side_by_side(t)
        else:
            down, mid = self.controlnet(self.model_input, t, self.ctx, self.cond, self.conditioning_scale,
                                        added_cond_kwargs=self.added, cond_embedding=self.cond_emb)
            self.unet.defer_conv_out = self.fuse_tail
            try:
                eps = self.unet(self.model_input, t, self.ctx, added_cond_kwargs=self.added,
                                down_block_additional_residuals=down, mid_block_additional_residual=mid,
                                return_dict=False)[0]
            finally:
                self.unet.defer_conv_out = False
        if self.fuse_tail:   # `eps` is the input of conv_out here
            ops.conv_out_cfg_euler(eps, self._co_w, self.unet.conv_out.bias, self.latents, self.row, self.guidance_scale,
                                   latents_out=self.latents, model_input_next=self.model_input)
        else:
            ops.cfg_euler_step(eps, self.latents, self.row, self.guidance_scale, latents_out=self.latents,
                               model_input_next=self.model_input)

    def _models_side_by_side(self, t):
        """The ControlNet on a second stream beside the UNet's down and mid blocks, which do not need its residuals:
        many of either model's launches leave CUs idle (160 tiles on 256 CUs) and every launch has a ramp and a tail.
        The counter arena is cleared once before the fork and neither forward resets it; the ControlNet's ops take a
        scratch buffer of their own; the UNet waits for the second stream right after its mid block."""
        from . import ops

        main = torch.cuda.current_stream()
        ops.split_counters_reset(self.latents.device)
        self._cn_stream.wait_stream(main)
        with ops.split_counters_held():
            with torch.cuda.stream(self._cn_stream), ops.side_branch():
                down, mid = self.controlnet(self.model_input, t, self.ctx, self.cond, self.conditioning_scale,
                                            added_cond_kwargs=self.added, cond_embedding=self.cond_emb)
            self.unet.defer_conv_out = self.fuse_tail
            self.unet.before_residuals = lambda: main.wait_stream(self._cn_stream)
            try:
                eps = self.unet(self.model_input, t, self.ctx, added_cond_kwargs=self.added,
                                down_block_additional_residuals=down, mid_block_additional_residual=mid,
                                return_dict=False)[0]
            finally:
                self.unet.defer_conv_out = False
                self.unet.before_residuals = None
        return eps

    def run(self, latents: torch.Tensor, scheduler, controlnet_cond: Optional[torch.Tensor] = None,
            check: bool = True, encoder_hidden_states: Optional[torch.Tensor] = None) -> torch.Tensor:
        """The whole loop: `latents` already scaled by init_noise_sigma (prepare_latents, pipeline :872-887);
        scheduler.set_timesteps(...) done.  Returns the final latents (a copy, in the model dtype like the reference's
        scheduler output, scheduling_euler_discrete.py:530)."""
        dev = self.latents.device
        table = torch.cat([scheduler.coef_table(dev), scheduler.timesteps.to(dev, torch.float32)[:, None]], dim=1).contiguous()
        with torch.no_grad():
            if controlnet_cond is not None:
                self.cond.copy_(controlnet_cond)
                if self.hoist:
                    self.cond_emb.copy_(self.controlnet.embed_condition(self.cond))
            if encoder_hidden_states is not None:
                self.ctx.copy_(encoder_hidden_states)
            self._project_context()
            self.latents.copy_(latents)
            self.model_input.copy_((torch.cat([latents] * 2).float() / table[0, 3]).to(torch.bfloat16))
            for i in range(table.shape[0]):
                self.row.copy_(table[i])
                self.graph.replay()
        if check:
            self._ops.check_split_timeouts(dev)
        return self.latents.clone()
