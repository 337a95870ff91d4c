"""The oracle's Euler scheduler against the reference's full-loop known answers
(diffusers-hf/tests/schedulers/test_scheduler_euler.py:51-161; harness inputs from
tests/schedulers/test_schedulers.py:341-368)."""
import pytest
import torch

from oracle.euler import EulerDiscreteScheduler, classifier_free_guidance, denoise_loop


def dummy_sample_deter():
    n = 4 * 3 * 8 * 8
    s = torch.arange(n).reshape(3, 8, 8, 4) / n
    return s.permute(3, 0, 1, 2)


def dummy_model(sample, t):
    t = t.reshape(-1, *(1,) * (sample.dim() - 1)).to(sample.dtype)
    return sample * t / (t + 1)


def full_loop(**cfg):
    sch = EulerDiscreteScheduler(num_train_timesteps=1100, beta_start=0.0001, beta_end=0.02, beta_schedule="linear", **cfg)
    sch.set_timesteps(10)
    sample = dummy_sample_deter() * sch.init_noise_sigma
    for t in sch.timesteps:
        sample = sch.scale_model_input(sample, t)
        sample = sch.step(dummy_model(sample, t), t, sample)
    return sample.abs().sum().item(), sample.abs().mean().item()


def test_full_loop_no_noise_kat():
    s, m = full_loop()
    assert abs(s - 10.0807) < 1e-2 and abs(m - 0.0131) < 1e-3


def test_full_loop_v_prediction_kat():
    s, m = full_loop(prediction_type="v_prediction")
    assert abs(s - 0.0002) < 1e-2 and abs(m - 2.2676e-06) < 1e-3


def test_full_loop_karras_kat():
    s, m = full_loop(use_karras_sigmas=True)
    assert abs(s - 124.52299499511719) < 1e-2 and abs(m - 0.16213932633399963) < 1e-3


def test_sdxl_schedule_shape():
    """SDXL's scheduler config: scaled_linear 0.00085..0.012, leading spacing, offset 1: 50 steps start at t = 981."""
    sch = EulerDiscreteScheduler(beta_start=0.00085, beta_end=0.012, beta_schedule="scaled_linear",
                                 timestep_spacing="leading", steps_offset=1)
    sch.set_timesteps(50)
    assert sch.timesteps[0].item() == 981.0 and sch.timesteps[-1].item() == 1.0 and len(sch.sigmas) == 51
    assert sch.sigmas[-1].item() == 0.0 and torch.all(sch.sigmas[:-1] > sch.sigmas[1:])
    # init_noise_sigma for "leading": sqrt(sigma_max^2 + 1)
    assert abs(sch.init_noise_sigma.item() - (sch.sigmas[0].item() ** 2 + 1) ** 0.5) < 1e-6


def test_guidance_and_loop_closed_forms():
    g = torch.Generator().manual_seed(0)
    n = torch.randn(2, 4, 8, 8, generator=g)
    assert torch.equal(classifier_free_guidance(n, 1.0), n[:1] + 1.0 * (n[1:] - n[:1]))
    assert torch.allclose(classifier_free_guidance(n, 0.0), n[:1])
    # a model that predicts zero noise leaves the latents unchanged by every Euler step
    sch = EulerDiscreteScheduler(beta_start=0.00085, beta_end=0.012, beta_schedule="scaled_linear",
                                 timestep_spacing="leading", steps_offset=1)
    sch.set_timesteps(5)
    lat = torch.randn(1, 4, 8, 8, generator=g)
    out = denoise_loop(lambda x, t: torch.zeros_like(x), sch, lat, 7.5)
    assert torch.equal(out, lat)
    # eps-prediction with the exact noise: x = x0 + sigma*eps, model returns eps -> one step lands on x0 + sigma_next*eps
    sch.set_timesteps(5)
    x0, eps = torch.randn(1, 4, 8, 8, generator=g), torch.randn(1, 4, 8, 8, generator=g)
    x = x0 + sch.sigmas[0] * eps
    t = sch.timesteps[0]
    sch.scale_model_input(x, t)
    nxt = sch.step(eps, t, x)
    assert torch.allclose(nxt, x0 + sch.sigmas[1] * eps, atol=1e-4)
