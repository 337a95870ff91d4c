"""ControlNet forward and the guided ControlNet + UNet denoise loop on the GPU against the CPU oracle
(tiny configuration: same topology as SDXL, small widths)."""
import pytest
import torch

from helpers import assert_close_rel, bf16_round, cosine, round_module_to_bf16_
from oracle.controlnet import ControlNetModel as OracleControlNet
from oracle.euler import EulerDiscreteScheduler as OracleScheduler, denoise_loop as oracle_loop
from oracle.unet_sdxl import UNet2DConditionModel as OracleUNet, UNetConfig as OracleCfg

pytestmark = pytest.mark.gpu
BF = torch.bfloat16
DEV = "cuda:0"


def say(*a):
    print(*a, flush=True)


def _randomise_zero_convs(cn, seed):
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for m in [cn.controlnet_cond_embedding.conv_out, cn.controlnet_mid_block, *cn.controlnet_down_blocks]:
            m.weight.copy_(torch.randn(m.weight.shape, generator=g) * (0.5 / m.weight[0].numel() ** 0.5))
            m.bias.copy_(torch.randn(m.bias.shape, generator=g) * 0.02)


def _inputs(cfg, H, S, seed):
    g = torch.Generator().manual_seed(seed)
    x = bf16_round(torch.randn(2, 4, H, H, generator=g))
    ctx = bf16_round(torch.randn(2, S, cfg.cross_attention_dim, generator=g))
    pooled = cfg.projection_class_embeddings_input_dim - 6 * cfg.addition_time_embed_dim
    added = dict(text_embeds=bf16_round(torch.randn(2, pooled, generator=g)),
                 time_ids=torch.tensor([[H * 8, H * 8, 0, 0, H * 8, H * 8]] * 2, dtype=torch.float32))
    cond = bf16_round(torch.rand(2, 3, H * 8, H * 8, generator=g))
    return x, ctx, added, cond


@pytest.fixture(scope="module")
def pair():
    import katz_amd.layers as L
    from katz_amd.controlnet import ControlNetModel
    from katz_amd.unet_2d_condition import UNet2DConditionModel, UNetConfig

    torch.manual_seed(0)
    cfg = OracleCfg.tiny()
    o_cn = OracleControlNet(cfg).eval()
    _randomise_zero_convs(o_cn, 1)
    round_module_to_bf16_(o_cn)
    o_unet = round_module_to_bf16_(OracleUNet(cfg).eval())
    L.SKIP_INIT = True
    try:
        p_cn, p_unet = ControlNetModel(UNetConfig.tiny()), UNet2DConditionModel(UNetConfig.tiny())
    finally:
        L.SKIP_INIT = False
    p_cn.load_state_dict(o_cn.state_dict(), strict=True)
    p_unet.load_state_dict(o_unet.state_dict(), strict=True)
    return cfg, o_cn, o_unet, p_cn.to_runtime(DEV, BF), p_unet.to_runtime(DEV, BF)


def test_controlnet_forward_matches_oracle(pair):
    cfg, o_cn, _, p_cn, _ = pair
    say("controlnet forward")
    x, ctx, added, cond = _inputs(cfg, 32, 77, 2)
    with torch.no_grad():
        rd, rm = o_cn(x, 500.0, ctx, cond, 0.5, added)
        gd, gm = p_cn(x.to(DEV), torch.tensor([500.0], device=DEV), ctx.to(DEV), cond.to(DEV), 0.5,
                      added_cond_kwargs={k: v.to(DEV) for k, v in added.items()})
    torch.cuda.synchronize()
    assert len(gd) == len(rd) == 9
    for j, (g, r) in enumerate(zip(gd + [gm], rd + [rm])):
        assert g.shape == r.shape
        assert cosine(g, r) >= 0.999, (j, cosine(g, r))
        # composite of up to ~40 bf16 layers: the contract is the cosine; the elementwise bound only catches gross errors
        assert_close_rel(g, r, 1e-1, f"controlnet residual {j}")
    # conditioning_scale is linear; Katz's default is 0.5 (controlnet.py:693)
    with torch.no_grad():
        gd1, _ = p_cn(x.to(DEV), torch.tensor([500.0], device=DEV), ctx.to(DEV), cond.to(DEV), 1.0,
                      added_cond_kwargs={k: v.to(DEV) for k, v in added.items()})
        gdd, _ = p_cn(x.to(DEV), torch.tensor([500.0], device=DEV), ctx.to(DEV), cond.to(DEV),
                      added_cond_kwargs={k: v.to(DEV) for k, v in added.items()})
    assert cosine(gd1[3].float() * 0.5, gd[3]) >= 0.9995 and cosine(gdd[3], gd[3]) >= 0.9995


def test_fresh_controlnet_is_exactly_zero():
    import katz_amd.layers as L
    from katz_amd.controlnet import ControlNetModel
    from katz_amd.unet_2d_condition import UNetConfig

    say("controlnet zeros")
    torch.manual_seed(3)
    cn = ControlNetModel(UNetConfig.tiny()).to_runtime(DEV, BF)
    cfg = OracleCfg.tiny()
    x, ctx, added, cond = _inputs(cfg, 16, 7, 4)
    with torch.no_grad():
        d, m = cn(x.to(DEV), 10.0, ctx.to(DEV), cond.to(DEV), added_cond_kwargs={k: v.to(DEV) for k, v in added.items()})
    assert all(torch.count_nonzero(t) == 0 for t in d) and torch.count_nonzero(m) == 0


def test_controlnet_unet_guided_loop_config5_shape(pair):
    """The whole configuration-5 loop at tiny widths: per step ControlNet -> UNet with its residuals ->
    guidance -> Euler, 6 steps, guidance 7.5, conditioning_scale 0.5, seeded latents x init_noise_sigma."""
    from katz_amd.scheduler import EulerDiscreteScheduler, denoise_loop

    cfg, o_cn, o_unet, p_cn, p_unet = pair
    say("config-5 loop")
    x, ctx, added, cond = _inputs(cfg, 16, 77, 5)
    sd = dict(beta_start=0.00085, beta_end=0.012, beta_schedule="scaled_linear", timestep_spacing="leading", steps_offset=1)
    osch, psch = OracleScheduler(**sd), EulerDiscreteScheduler(**sd)
    osch.set_timesteps(6)
    psch.set_timesteps(6, device=DEV)
    lat0 = bf16_round(x[:1] * osch.init_noise_sigma)
    added_d = {k: v.to(DEV) for k, v in added.items()}

    def o_model(inp, t):
        with torch.no_grad():
            inp = bf16_round(inp)
            d, m = o_cn(inp, t, ctx, cond, 0.5, added)
            return bf16_round(o_unet(inp, t, ctx, added, [bf16_round(v) for v in d], bf16_round(m)))

    def p_model(inp, t):
        with torch.no_grad():
            d, m = p_cn(inp, t.reshape(1), ctx.to(DEV), cond.to(DEV), 0.5, added_cond_kwargs=added_d)
            return p_unet(inp, t.reshape(1), ctx.to(DEV), added_cond_kwargs=added_d, down_block_additional_residuals=d,
                          mid_block_additional_residual=m, return_dict=False)[0]

    ref = oracle_loop(o_model, osch, lat0.float(), 7.5)
    got = denoise_loop(p_model, psch, lat0.to(DEV), 7.5, latents_fp32=True)
    torch.cuda.synchronize()
    assert got.shape == ref.shape == (1, 4, 16, 16)
    assert torch.isfinite(got).all()
    assert cosine(got, ref) >= 0.999, cosine(got, ref)
