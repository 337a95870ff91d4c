"""CPU restatement of the reference's Euler discrete scheduler and the CFG combination of the denoise loop.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).  Follows
diffusers-hf/src/diffusers/schedulers/scheduling_euler_discrete.py (constructor :177-236,
init_noise_sigma :241-247, scale_model_input :274-298, set_timesteps :300-362, Karras sigmas :387-410,
index_for_timestep / _init_step_index :412-434, step :435-545 with s_churn = 0) and the guidance lines of
diffusers-hf/src/diffusers/pipelines/controlnet/pipeline_controlnet_sd_xl_katz.py:1565-1570, :1647-1658.

Pinned by the reference's full-loop known answers (tests/schedulers/test_scheduler_euler.py:51-77 epsilon,
:79-105 v_prediction, :107-133 device variant, :135-161 Karras sigmas) in tests/test_oracle_euler.py.

sigmas are kept as 0-dim fp32 tensors exactly as the reference keeps them, so torch's type promotion
(a 0-dim fp32 tensor does not promote a half tensor) rounds where the reference rounds.  One thing is spelled
out by hand: the reference runs on the GPU, where a 0-dim CPU scalar enters an elementwise kernel as an fp32
value (`half_tensor * sigma` = round_half(float(x) * sigma)); the CPU kernels instead round the scalar to half
first.  `_scalar_op` evaluates such products / quotients the GPU way so that the oracle follows the reference
as it runs, not a CPU artefact.  For fp32 tensors (all known-answer tests) both are the same operation.
"""
from __future__ import annotations

import numpy as np
import torch


def _scalar_op(x: torch.Tensor, scalar: torch.Tensor, op) -> torch.Tensor:
    """op(x, 0-dim fp32 scalar) with the scalar kept in fp32 and the result rounded to x's dtype."""
    if x.dtype == torch.float32:
        return op(x, scalar)
    return op(x.float(), scalar).to(x.dtype)


class EulerDiscreteScheduler:
    order = 1

    def __init__(self, num_train_timesteps: int = 1000, beta_start: float = 0.0001, beta_end: float = 0.02,
                 beta_schedule: str = "linear", prediction_type: str = "epsilon", use_karras_sigmas: bool = False,
                 timestep_spacing: str = "linspace", steps_offset: int = 0):
        if beta_schedule == "linear":
            betas = torch.linspace(beta_start, beta_end, num_train_timesteps, dtype=torch.float32)
        elif beta_schedule == "scaled_linear":
            betas = torch.linspace(beta_start ** 0.5, beta_end ** 0.5, num_train_timesteps, dtype=torch.float32) ** 2
        else:
            raise NotImplementedError(beta_schedule)
        self.num_train_timesteps = num_train_timesteps
        self.prediction_type = prediction_type
        self.use_karras_sigmas = use_karras_sigmas
        self.timestep_spacing = timestep_spacing
        self.steps_offset = steps_offset
        self.alphas_cumprod = torch.cumprod(1.0 - betas, dim=0)
        sigmas = (((1 - self.alphas_cumprod) / self.alphas_cumprod) ** 0.5).flip(0)
        self.timesteps = torch.from_numpy(np.linspace(0, num_train_timesteps - 1, num_train_timesteps, dtype=float)[::-1].copy()).to(torch.float32)
        self.sigmas = torch.cat([sigmas, torch.zeros(1)])
        self.step_index = None

    @property
    def init_noise_sigma(self):
        max_sigma = self.sigmas.max()
        if self.timestep_spacing in ("linspace", "trailing"):
            return max_sigma
        return (max_sigma ** 2 + 1) ** 0.5

    def set_timesteps(self, num_inference_steps: int):
        n_train = self.num_train_timesteps
        if self.timestep_spacing == "linspace":
            timesteps = np.linspace(0, n_train - 1, num_inference_steps, dtype=np.float32)[::-1].copy()
        elif self.timestep_spacing == "leading":
            step_ratio = n_train // num_inference_steps
            timesteps = (np.arange(0, num_inference_steps) * step_ratio).round()[::-1].copy().astype(np.float32)
            timesteps += self.steps_offset
        elif self.timestep_spacing == "trailing":
            step_ratio = n_train / num_inference_steps
            timesteps = (np.arange(n_train, 0, -step_ratio)).round().copy().astype(np.float32)
            timesteps -= 1
        else:
            raise ValueError(self.timestep_spacing)
        sigmas = (((1 - self.alphas_cumprod) / self.alphas_cumprod) ** 0.5).numpy()
        log_sigmas = np.log(sigmas)
        sigmas = np.interp(timesteps, np.arange(0, len(sigmas)), sigmas)
        if self.use_karras_sigmas:
            sigmas = self._convert_to_karras(sigmas, num_inference_steps)
            timesteps = np.array([self._sigma_to_t(s, log_sigmas) for s in sigmas])
        sigmas = torch.from_numpy(sigmas).to(dtype=torch.float32)
        self.timesteps = torch.from_numpy(timesteps.astype(np.float32))
        self.sigmas = torch.cat([sigmas, torch.zeros(1)])
        self.step_index = None

    @staticmethod
    def _sigma_to_t(sigma, log_sigmas):
        log_sigma = np.log(np.maximum(sigma, 1e-10))
        dists = log_sigma - log_sigmas[:, np.newaxis]
        low_idx = np.cumsum((dists >= 0), axis=0).argmax(axis=0).clip(max=log_sigmas.shape[0] - 2)
        high_idx = low_idx + 1
        low, high = log_sigmas[low_idx], log_sigmas[high_idx]
        w = np.clip((low - log_sigma) / (low - high), 0, 1)
        return ((1 - w) * low_idx + w * high_idx).reshape(np.shape(sigma))

    @staticmethod
    def _convert_to_karras(in_sigmas, num_inference_steps):
        sigma_min, sigma_max = in_sigmas[-1].item(), in_sigmas[0].item()
        rho = 7.0
        ramp = np.linspace(0, 1, num_inference_steps)
        min_inv_rho, max_inv_rho = sigma_min ** (1 / rho), sigma_max ** (1 / rho)
        return (max_inv_rho + ramp * (min_inv_rho - max_inv_rho)) ** rho

    def _init_step_index(self, timestep):
        indices = (self.timesteps == timestep).nonzero()
        pos = 1 if len(indices) > 1 else 0
        self.step_index = indices[pos].item()

    def scale_model_input(self, sample: torch.Tensor, timestep) -> torch.Tensor:
        if self.step_index is None:
            self._init_step_index(timestep)
        sigma = self.sigmas[self.step_index]
        return _scalar_op(sample, (sigma ** 2 + 1) ** 0.5, torch.div)

    def step(self, model_output: torch.Tensor, timestep, sample: torch.Tensor) -> torch.Tensor:
        if self.step_index is None:
            self._init_step_index(timestep)
        sample = sample.to(torch.float32)
        sigma = self.sigmas[self.step_index]
        sigma_hat = sigma * (0.0 + 1)  # gamma = 0 (s_churn = 0)
        if self.prediction_type == "epsilon":
            pred_original_sample = sample - _scalar_op(model_output, sigma_hat, torch.mul)
        elif self.prediction_type == "v_prediction":
            pred_original_sample = _scalar_op(model_output, -sigma / (sigma ** 2 + 1) ** 0.5, torch.mul) + (sample / (sigma ** 2 + 1))
        else:
            raise ValueError(self.prediction_type)
        derivative = (sample - pred_original_sample) / sigma_hat
        dt = self.sigmas[self.step_index + 1] - sigma_hat
        prev_sample = (sample + derivative * dt).to(model_output.dtype)
        self.step_index += 1
        return prev_sample


def classifier_free_guidance(noise_pred: torch.Tensor, guidance_scale: float) -> torch.Tensor:
    """pipeline_controlnet_sd_xl_katz.py:1649-1650: rows [uncond; text] -> uncond + g * (text - uncond), in the
    dtype of noise_pred."""
    noise_pred_uncond, noise_pred_text = noise_pred.chunk(2)
    return noise_pred_uncond + guidance_scale * (noise_pred_text - noise_pred_uncond)


def denoise_loop(model, scheduler: EulerDiscreteScheduler, latents: torch.Tensor, guidance_scale: float):
    """The loop body of pipeline_controlnet_sd_xl_katz.py:1509-1658 around a model callable
    model(latent_model_input [2B,...], t) -> noise_pred [2B,...]: duplicate, scale, predict, guide, step."""
    for t in scheduler.timesteps:
        latent_model_input = torch.cat([latents] * 2)
        latent_model_input = scheduler.scale_model_input(latent_model_input, t)
        noise_pred = model(latent_model_input, t)
        noise_pred = classifier_free_guidance(noise_pred, guidance_scale)
        latents = scheduler.step(noise_pred, t, latents)
    return latents
