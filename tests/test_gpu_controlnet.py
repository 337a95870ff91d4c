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


def test_graphed_denoise_step_matches_eager_loop(pair):
    """ControlNet -> UNet -> guidance + Euler as one captured graph per step (GraphedDenoiseStep) against the same
    loop run eagerly, kernel by kernel: identical latents bit for bit, also on a second run with other latents, with
    the conditioning embedding hoisted out of the loop or recomputed inside the graph, and with the ControlNet on a
    second stream beside the UNet's down blocks (the default) or in front of the UNet on one stream."""
    from katz_amd.graph import GraphedDenoiseStep
    from katz_amd.scheduler import EulerDiscreteScheduler, denoise_loop

    cfg, _, _, p_cn, p_unet = pair
    say("graphed denoise step")
    x, ctx, added, cond = _inputs(cfg, 16, 77, 7)
    psch = EulerDiscreteScheduler(beta_start=0.00085, beta_end=0.012, beta_schedule="scaled_linear",
                                  timestep_spacing="leading", steps_offset=1)
    psch.set_timesteps(5, device=DEV)
    added_d = {k: v.to(DEV) for k, v in added.items()}

    def p_model(inp, t):
        with torch.no_grad():
            d, m = p_cn(inp, t.reshape(1), ctx.to(DEV), cond.to(DEV), 0.5, added_cond_kwargs=added_d)
            return p_unet(inp, t.reshape(1), ctx.to(DEV), added_cond_kwargs=added_d, down_block_additional_residuals=d,
                          mid_block_additional_residual=m, return_dict=False)[0]

    lats = [bf16_round(x[:1] * psch.init_noise_sigma), bf16_round(x[1:] * psch.init_noise_sigma)]
    eager = [denoise_loop(p_model, psch, l.to(DEV), 7.5) for l in lats]
    for hoist, fuse_tail, overlap in ((True, False, True), (False, False, True), (True, True, True),
                                      (True, False, False), (False, False, False)):
        step = GraphedDenoiseStep(p_unet, p_cn, lats[0].to(DEV), ctx.to(DEV), added_d, cond.to(DEV), 7.5, 0.5,
                                  hoist_cond_embedding=hoist, fuse_tail=fuse_tail, overlap=overlap)
        assert step.fuse_tail == fuse_tail and step.overlap == overlap
        for l, e in zip(lats, eager):
            got = step.run(l.to(DEV), psch)
            torch.cuda.synchronize()
            assert got.shape == e.shape and torch.isfinite(got).all()
            if not fuse_tail:   # the same kernels in the same order: the same bits
                assert torch.equal(got.contiguous(), e.contiguous()), (hoist, (got.float() - e.float()).abs().max().item())
            else:               # conv_out inside the scheduler kernel sums its taps in another order: last-bit noise,
                                # amplified by five steps of a random-weight network
                assert cosine(got, e) >= 0.9995, cosine(got, e)


def test_config5_loop_with_two_loras_against_the_oracle_loop():
    """Configuration 5 with its adapters at tiny widths: ControlNet -> UNet carrying TWO active LoRAs (weights 0.8 / 0.6)
    -> guidance 7.5 -> Euler, 6 steps, against oracle.euler.denoise_loop over the oracle models with the same adapters:
    the eager loop, and GraphedDenoiseStep (one graph per step, conv_out + guidance + Euler fused) with the ControlNet
    beside the UNet's down blocks on a second stream and in front of it on one stream.  Cosine >= 0.999 each; the two
    graph forms agree bit for bit, and the unfused graph equals the eager loop bit for bit."""
    import katz_amd.layers as L
    from katz_amd import ops
    from katz_amd.controlnet import ControlNetModel
    from katz_amd.graph import GraphedDenoiseStep
    from katz_amd.scheduler import EulerDiscreteScheduler, denoise_loop
    from katz_amd.unet_2d_condition import UNet2DConditionModel, UNetConfig

    say("config-5 loop with two LoRAs")
    torch.manual_seed(4)
    cfg = OracleCfg.tiny()
    o_cn = OracleControlNet(cfg).eval()
    _randomise_zero_convs(o_cn, 2)
    round_module_to_bf16_(o_cn)
    o_unet = round_module_to_bf16_(OracleUNet(cfg).eval())
    L.SKIP_INIT = True
    try:
        p_cn, p_unet = ControlNetModel(UNetConfig.tiny()), UNet2DConditionModel(UNetConfig.tiny())
    finally:
        L.SKIP_INIT = False
    p_cn.load_state_dict(o_cn.state_dict(), strict=True)
    p_unet.load_state_dict(o_unet.state_dict(), strict=True)
    p_cn, p_unet = p_cn.to_runtime(DEV, BF), p_unet.to_runtime(DEV, BF)
    g = torch.Generator().manual_seed(11)
    lora = {}
    for name, m in o_unet.lora_linears().items():
        for an, r in (("r16", 16), ("r8", 8)):
            d = bf16_round(torch.randn(r, m.in_features, generator=g) * 0.05)
            u = bf16_round(torch.randn(m.out_features, r, generator=g) * 0.05)
            m.add_adapter(an, d, u)
            lora.setdefault(an, {})[f"unet.{name}.lora.down.weight"] = d
            lora[an][f"unet.{name}.lora.up.weight"] = u
    o_unet.set_adapters(["r16", "r8"], [0.8, 0.6])
    for an in ("r16", "r8"):
        p_unet.load_lora_into_unet(lora[an], adapter_name=an)
    p_unet.set_adapters(["r16", "r8"], [0.8, 0.6])

    x, ctx, added, cond = _inputs(cfg, 16, 77, 12)
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
    # the adapters matter: without them the oracle loop ends somewhere else
    o_unet.set_adapters([], [])
    osch.set_timesteps(6)                   # a fresh step index for the second loop
    ref_free = oracle_loop(o_model, osch, lat0.float(), 7.5)
    o_unet.set_adapters(["r16", "r8"], [0.8, 0.6])
    assert cosine(ref_free, ref) < 0.9999, cosine(ref_free, ref)
    eager = denoise_loop(p_model, psch, lat0.to(DEV), 7.5)
    torch.cuda.synchronize()
    assert torch.isfinite(eager).all() and cosine(eager, ref) >= 0.999, cosine(eager, ref)
    got = {}
    for overlap in (True, False):
        for fuse_tail in (True, False):
            step = GraphedDenoiseStep(p_unet, p_cn, lat0.to(DEV), ctx.to(DEV), added_d, cond.to(DEV), 7.5, 0.5,
                                      fuse_tail=fuse_tail, overlap=overlap)
            assert step.overlap == overlap and step.fuse_tail == fuse_tail
            out = step.run(lat0.to(DEV), psch)          # raises if an in-launch shrink wait ran out
            again = step.run(lat0.to(DEV), psch)
            torch.cuda.synchronize()
            assert torch.isfinite(out).all() and torch.equal(out, again)
            assert cosine(out, ref) >= 0.999, (overlap, fuse_tail, cosine(out, ref))
            got[(overlap, fuse_tail)] = out
    assert torch.equal(got[(True, True)], got[(False, True)]) and torch.equal(got[(True, False)], got[(False, False)])
    # the context K / V projected inside every step (as the reference does) instead of once per loop: the same bits
    in_step = GraphedDenoiseStep(p_unet, p_cn, lat0.to(DEV), ctx.to(DEV), added_d, cond.to(DEV), 7.5, 0.5,
                                 hoist_context_kv=False).run(lat0.to(DEV), psch)
    assert torch.equal(in_step, got[(True, True)])
    assert torch.equal(got[(True, False)].contiguous(), eager.contiguous())
    ops.check_split_timeouts(torch.device(DEV))


def test_sdxl_size_controlnet_forward_and_step():
    """ONE full-size ControlNet forward (SDXL widths, conditioning image [2,3,1024,1024], latents [2,4,128,128]) feeding
    one full-size UNet step WITH configuration 5's two adapters (rank 64 weight 0.8 + rank 32 weight 0.6 on all 722
    linears): residual shapes of unet_2d_condition.py:539-563, finite values, bit-reproducible, the adapters change the
    result, and the captured ControlNet -> UNet -> guidance + Euler graph equal to the eager sequence (the ControlNet
    beside the UNet's in-launch-shrink kernels on a second stream, or in front of them).  Random-init weights, the
    ControlNet built with from_unet and non-zero "zero" convolutions; no oracle at this size (the CPU model needs
    minutes), parity of the same code is checked at small widths above and against the reference's own outputs in
    test_gpu_reference_fixture.py."""
    import katz_amd.layers as L
    from katz_amd import ops
    from katz_amd.controlnet import ControlNetModel
    from katz_amd.graph import GraphedDenoiseStep
    from katz_amd.scheduler import EulerDiscreteScheduler
    from katz_amd.unet_2d_condition import UNet2DConditionModel, UNetConfig

    say("sdxl-size controlnet + unet step")
    torch.manual_seed(0)
    with torch.device(DEV):
        unet = UNet2DConditionModel(UNetConfig.sdxl())
        cn = ControlNetModel.from_unet(unet)
        g = torch.Generator(device=DEV).manual_seed(1)
        with torch.no_grad():
            for m in [cn.controlnet_cond_embedding.conv_out, cn.controlnet_mid_block, *cn.controlnet_down_blocks]:
                m.weight.copy_(torch.randn(m.weight.shape, generator=g, device=DEV) * (0.5 / m.weight[0].numel() ** 0.5))
    unet, cn = unet.to_runtime(DEV, BF), cn.to_runtime(DEV, BF)
    rn = lambda *s: torch.randn(*s, generator=g, device=DEV).to(BF)
    lins = unet.lora_linears()
    assert len(lins) == 722
    for name, rank in (("r64", 64), ("r32", 32)):
        for lin in lins.values():
            lin.add_adapter(name, (rn(rank, lin.in_features).float() * 0.02).to(BF),
                            (rn(lin.out_features, rank).float() * 0.02).to(BF), alpha=None)
    lat = rn(1, 4, 128, 128)
    x = torch.cat([lat, lat])
    ctx = rn(2, 77, 2048)
    added = dict(text_embeds=rn(2, 1280), time_ids=torch.tensor([[1024.0, 1024, 0, 0, 1024, 1024]] * 2, device=DEV))
    cond = torch.rand(2, 3, 1024, 1024, generator=g, device=DEV).to(BF)
    t = torch.tensor([500.0], device=DEV)
    with torch.no_grad():
        d, m = cn(x, t, ctx, cond, 0.5, added_cond_kwargs=added)
        d2, m2 = cn(x, t, ctx, cond, 0.5, added_cond_kwargs=added)
        shapes = [(320, 128)] * 3 + [(320, 64), (640, 64), (640, 64), (640, 32), (1280, 32), (1280, 32)]
        assert [tuple(r.shape) for r in d] == [(2, c, h, h) for c, h in shapes] and tuple(m.shape) == (2, 1280, 32, 32)
        for a, b in zip(list(d) + [m], list(d2) + [m2]):
            assert torch.isfinite(a).all() and torch.equal(a, b)
            assert a.float().abs().max() > 0
        eps_free = unet(x, t, ctx, added_cond_kwargs=added, down_block_additional_residuals=d, mid_block_additional_residual=m).sample
        unet.set_adapters(["r64", "r32"], [0.8, 0.6])
        eps = unet(x, t, ctx, added_cond_kwargs=added, down_block_additional_residuals=d, mid_block_additional_residual=m).sample
        assert eps.shape == (2, 4, 128, 128) and torch.isfinite(eps).all() and torch.isfinite(eps_free).all()
        assert not torch.equal(eps, eps_free) and cosine(eps, eps_free) > 0.5     # the adapters are in the step
        # one step of the loop: eager sequence against the captured graph
        sch = EulerDiscreteScheduler(beta_start=0.00085, beta_end=0.012, beta_schedule="scaled_linear",
                                     timestep_spacing="leading", steps_offset=1)
        sch.set_timesteps(2, device=DEV)
        lat0 = (lat.float() * sch.init_noise_sigma).to(BF)
        step = GraphedDenoiseStep(unet, cn, lat0, ctx, added, cond, 7.5, 0.5, fuse_tail=False)
        assert step.overlap
        got = step.run(lat0, sch)
        fused = GraphedDenoiseStep(unet, cn, lat0, ctx, added, cond, 7.5, 0.5).run(lat0, sch)   # conv_out inside the step kernel
        one_stream = GraphedDenoiseStep(unet, cn, lat0, ctx, added, cond, 7.5, 0.5, overlap=False).run(lat0, sch)
        assert torch.equal(fused, one_stream)   # the ControlNet beside the down blocks or in front of them: the same bits
        coef = sch.coef_table(DEV)
        cur = lat0.contiguous(memory_format=torch.channels_last)
        inp = (torch.cat([cur] * 2).float() / coef[0, 3]).to(BF).contiguous(memory_format=torch.channels_last)
        for i in range(2):
            ti = sch.timesteps[i].to(DEV, torch.float32).reshape(1)
            dd, mm = cn(inp, ti, ctx, cond, 0.5, added_cond_kwargs=added)
            e = unet(inp, ti, ctx, added_cond_kwargs=added, down_block_additional_residuals=dd, mid_block_additional_residual=mm).sample
            nxt = torch.empty_like(inp)
            cur = ops.cfg_euler_step(e, cur, coef[i], 7.5, model_input_next=nxt)
            inp = nxt
        torch.cuda.synchronize()
        assert torch.isfinite(got).all() and torch.equal(got, cur)
        assert torch.isfinite(fused).all() and cosine(fused, cur) >= 0.9999, cosine(fused, cur)
    ops.check_split_timeouts(torch.device(DEV))


def test_two_stream_helpers_keep_scratch_apart():
    """What lets two models run side by side on two streams: inside split_counters_held() a reset neither clears the
    counter arena nor hands its slices out again; inside side_branch() the shared GroupNorm scratch is another buffer."""
    from katz_amd import ops

    dev = torch.device(DEV)
    ops.split_counters_reset(dev)
    a = ops._arena_ints(dev, 4)
    a.fill_(7)
    with ops.split_counters_held():
        ops.split_counters_reset(dev)            # what a model's forward does at its start
        b = ops._arena_ints(dev, 4)
        assert a.tolist() == [7, 7, 7, 7] and b.tolist() == [0, 0, 0, 0]
        assert b.data_ptr() == a.data_ptr() + 16
    ops.split_counters_reset(dev)
    c = ops._arena_ints(dev, 4)
    assert c.data_ptr() == a.data_ptr() and c.tolist() == [0, 0, 0, 0]
    main_ws = ops._workspace(1024, dev)
    with ops.side_branch():
        side_ws = ops._workspace(1024, dev)
        assert side_ws.data_ptr() != main_ws.data_ptr()
        assert ops._workspace(1024, dev).data_ptr() == side_ws.data_ptr()
    assert ops._workspace(1024, dev).data_ptr() == main_ws.data_ptr()
    ops.split_counters_reset(dev)
