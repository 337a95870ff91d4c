"""Euler discrete scheduler and the guided denoise loop around the UNet step.

Host-side mirror of the reference's `EulerDiscreteScheduler`
(diffusers-hf/src/diffusers/schedulers/scheduling_euler_discrete.py: constructor :177-236, set_timesteps
:300-362, scale_model_input :274-298, step :435-545) with the same method names, plus `coef_table`, which feeds
the fused guidance + Euler kernel (`ops.cfg_euler_step`).  The schedule (a few hundred floats) is computed
on the host with numpy in the reference's order of operations; all per-element work runs on the GPU.
"""
from __future__ import annotations

from typing import Callable, Optional

import numpy as np
import torch

from . import ops


class EulerDiscreteScheduler:
    order = 1

    def __init__(self, num_train_timesteps: int = 1000, beta_start: float = 0.0001, beta_end: float = 0.02,
                 beta_schedule: str = "linear", prediction_type: str = "epsilon", timestep_spacing: str = "linspace",
                 steps_offset: int = 0):
        # torch's fp32 linspace / cumprod on the host, as the reference computes them (same roundings)
        if beta_schedule == "linear":
            betas = torch.linspace(beta_start, beta_end, num_train_timesteps, dtype=torch.float32)
        elif beta_schedule == "scaled_linear":
            betas = torch.linspace(beta_start ** 0.5, beta_end ** 0.5, num_train_timesteps, dtype=torch.float32) ** 2
        else:
            raise NotImplementedError(f"{beta_schedule} is not implemented for {self.__class__.__name__}")
        if prediction_type != "epsilon":
            raise NotImplementedError("only epsilon prediction (SDXL) is built")
        if timestep_spacing not in ("linspace", "leading", "trailing"):
            raise ValueError(f"{timestep_spacing} is not supported")
        self.num_train_timesteps, self.timestep_spacing, self.steps_offset = num_train_timesteps, timestep_spacing, steps_offset
        self.prediction_type = prediction_type
        self.alphas_cumprod = torch.cumprod(1.0 - betas, dim=0)
        self._train_sigmas = (((1 - self.alphas_cumprod) / self.alphas_cumprod) ** 0.5).numpy()
        self.sigmas = torch.from_numpy(np.concatenate([self._train_sigmas[::-1], np.zeros(1, np.float32)]).copy())
        self.timesteps = torch.from_numpy(np.linspace(0, num_train_timesteps - 1, num_train_timesteps, dtype=float)[::-1].copy()).float()
        self.num_inference_steps = None
        self._step_index = None

    @classmethod
    def sdxl(cls) -> "EulerDiscreteScheduler":
        """The scheduler configuration SDXL base ships (scaled_linear 0.00085..0.012, leading spacing, offset 1)."""
        return cls(beta_start=0.00085, beta_end=0.012, beta_schedule="scaled_linear", timestep_spacing="leading", steps_offset=1)

    @property
    def init_noise_sigma(self) -> torch.Tensor:
        max_sigma = self.sigmas.max()
        return max_sigma if self.timestep_spacing in ("linspace", "trailing") else (max_sigma ** 2 + 1) ** 0.5

    @property
    def step_index(self):
        return self._step_index

    def set_timesteps(self, num_inference_steps: int, device=None) -> None:
        n_train = self.num_train_timesteps
        self.num_inference_steps = num_inference_steps
        if self.timestep_spacing == "linspace":
            timesteps = np.linspace(0, n_train - 1, num_inference_steps, dtype=np.float32)[::-1].copy()
        elif self.timestep_spacing == "leading":
            timesteps = (np.arange(0, num_inference_steps) * (n_train // num_inference_steps)).round()[::-1].copy().astype(np.float32)
            timesteps += self.steps_offset
        else:
            timesteps = np.arange(n_train, 0, -n_train / num_inference_steps).round().copy().astype(np.float32) - 1
        sigmas = np.interp(timesteps, np.arange(0, len(self._train_sigmas)), self._train_sigmas).astype(np.float32)
        self.timesteps = torch.from_numpy(timesteps).to(device=device)
        self.sigmas = torch.from_numpy(np.concatenate([sigmas, np.zeros(1, np.float32)]))  # on the host, like the reference
        self._step_index = None

    def _init_step_index(self, timestep) -> None:
        t = timestep.item() if isinstance(timestep, torch.Tensor) else float(timestep)
        idx = (self.timesteps.cpu() == t).nonzero()
        self._step_index = idx[1 if len(idx) > 1 else 0].item()

    def scale_model_input(self, sample: torch.Tensor, timestep) -> torch.Tensor:
        if self._step_index is None:
            self._init_step_index(timestep)
        sigma = self.sigmas[self._step_index]
        return sample / ((sigma ** 2 + 1) ** 0.5)

    def step(self, model_output: torch.Tensor, timestep, sample: torch.Tensor, return_dict: bool = False):
        """Unfused form (torch elementwise ops), for callers that drive the scheduler as the reference does."""
        if self._step_index is None:
            self._init_step_index(timestep)
        sample = sample.to(torch.float32)
        sigma = self.sigmas[self._step_index]
        pred_original_sample = sample - sigma * model_output
        derivative = (sample - pred_original_sample) / sigma
        prev_sample = (sample + derivative * (self.sigmas[self._step_index + 1] - sigma)).to(model_output.dtype)
        self._step_index += 1
        return (prev_sample,)

    def coef_table(self, device) -> torch.Tensor:
        """[steps, 4] fp32 on `device`: {sigma_i, sigma_{i+1}, sqrt(sigma_{i+1}^2 + 1), sqrt(sigma_i^2 + 1)}: row i is
        what the fused step kernel reads at step i."""
        s = self.sigmas.numpy().astype(np.float32)
        nxt = (s[1:] * s[1:] + np.float32(1)) ** np.float32(0.5)
        cur = (s[:-1] * s[:-1] + np.float32(1)) ** np.float32(0.5)
        return torch.from_numpy(np.stack([s[:-1], s[1:], nxt, cur], axis=1).astype(np.float32)).to(device)


def denoise_loop(model: Callable[[torch.Tensor, torch.Tensor], torch.Tensor], scheduler: EulerDiscreteScheduler,
                 latents: torch.Tensor, guidance_scale: float, latents_fp32: bool = False,
                 check: bool = True) -> torch.Tensor:
    """The guided denoise loop of the reference (pipeline_controlnet_sd_xl_katz.py:1509-1658) around
    model(latent_model_input [2B,...] bf16, t) -> noise_pred [2B,...] bf16, with guidance, the Euler update and
    the next step's input scaling fused into one kernel per step.  `latents` must already be scaled by
    init_noise_sigma (prepare_latents, :872-887).  latents_fp32 keeps the latents in fp32 between steps
    instead of the model dtype the reference casts them to.  check: wait for the loop at its end and raise if a
    bounded in-launch wait of the LoRA linears ran out on the way (ops.check_split_timeouts)."""
    dev = latents.device
    coef = scheduler.coef_table(dev)
    lat = latents.to(torch.float32 if latents_fp32 else torch.bfloat16).contiguous()
    x = torch.cat([lat] * 2).to(torch.bfloat16)
    # first scale_model_input (later ones come out of the fused kernel): the division in fp32, as the reference's
    # `sample / ((sigma**2 + 1) ** 0.5)` with its CPU-resident sigma evaluates it (scheduling_euler_discrete.py:292-296)
    model_input = (x.float() / coef[0, 3]).to(torch.bfloat16).contiguous()
    nxt = torch.empty_like(model_input)
    lat_out = torch.empty_like(lat)
    timesteps = scheduler.timesteps.to(dev)
    for i in range(len(timesteps)):
        noise_pred = model(model_input, timesteps[i])
        ops.cfg_euler_step(noise_pred.contiguous(), lat, coef[i], guidance_scale, latents_out=lat_out, model_input_next=nxt)
        lat, lat_out = lat_out, lat
        model_input, nxt = nxt, model_input
    if check and dev.type == "cuda":
        ops.check_split_timeouts(dev)
    return lat
