"""Host-side logic that needs no GPU: imports, LoRA key parsing, adapter packing, state-dict hooks."""
import torch

from helpers import katz_lora_state_dict


def test_package_imports_without_gpu():
    import katz_amd.graph  # noqa: F401
    import katz_amd.layers  # noqa: F401
    import katz_amd.lora  # noqa: F401
    import katz_amd.ops  # noqa: F401
    import katz_amd.unet_2d_condition  # noqa: F401
    import katz_amd.unet_blocks  # noqa: F401


def test_ops_fail_loudly_without_gpu():
    """No CPU fallback: a CPU tensor is rejected with an explicit error."""
    import pytest
    from katz_amd import _lib, ops

    if not _lib.LIB_PATH.exists():
        pytest.skip("libkatz_hip.so not built")
    x = torch.zeros(4, 8, dtype=torch.bfloat16)
    with pytest.raises(_lib.KatzHipError):
        ops.lora_linear(x, torch.zeros(8, 8, dtype=torch.bfloat16))
    with pytest.raises(_lib.KatzHipError):
        ops.group_norm(torch.zeros(1, 8, 2, 2, dtype=torch.bfloat16), 2, None, None, 1e-5)


def test_parse_lora_key_spellings():
    from katz_amd.unet_2d_condition import parse_lora_key

    base = "down_blocks.1.attentions.0.transformer_blocks.0"
    assert parse_lora_key(f"unet.{base}.attn1.processor.to_q_lora.down.weight") == (f"{base}.attn1.to_q", "down")
    assert parse_lora_key(f"unet.{base}.attn2.processor.to_out_lora.up.weight") == (f"{base}.attn2.to_out.0", "up")
    assert parse_lora_key(f"unet.{base}.ff.net.0.proj.lora.down.weight") == (f"{base}.ff.net.0.proj", "down")
    assert parse_lora_key(f"{base}.ff.net.2.lora_A.weight") == (f"{base}.ff.net.2", "down")
    assert parse_lora_key(f"{base}.attn1.to_v.lora_B.default_0.weight") == (f"{base}.attn1.to_v", "up")
    assert parse_lora_key("text_encoder.something.weight") is None


def test_every_reference_lora_key_resolves_to_a_module():
    """All 1444 down/up keys of the reference's adapter metadata parse to one of the 722 LoRA linears."""
    import json
    from pathlib import Path

    import katz_amd.layers as L
    from katz_amd.unet_2d_condition import UNet2DConditionModel, UNetConfig, parse_lora_key

    keys = json.loads((Path(__file__).parent / "golden" / "sdxl_lora_keys.json").read_text())
    L.SKIP_INIT = True
    try:
        with torch.device("meta"):
            unet = UNet2DConditionModel(UNetConfig.sdxl())
    finally:
        L.SKIP_INIT = False
    lin = unet.lora_linears()
    assert len(lin) == 722
    for unet_key, meta in keys.items():
        mod = unet_key[: -len(".weight")]
        assert parse_lora_key(meta["down_key"]) == (mod, "down")
        assert parse_lora_key(meta["up_key"]) == (mod, "up")
        assert (lin[mod].in_features, lin[mod].out_features) == (meta["down"][1], meta["up"][0])


def test_pack_adapters_layout_and_rescale():
    from katz_amd.lora import Adapter, interleave_geglu_rows, pack_adapters, rescale_

    g = torch.Generator().manual_seed(0)
    ads = {"a": Adapter(torch.randn(8, 16, generator=g), torch.randn(64, 8, generator=g), alpha=16.0, weight=0.5),
           "b": Adapter(torch.randn(4, 16, generator=g), torch.randn(64, 4, generator=g), alpha=None, weight=2.0)}
    pk = pack_adapters(ads, ["b", "a"], 16, 64, torch.float32, "cpu", global_scale=0.5)
    assert pk.R == 64 and pk.a_cat.shape == (64, 16) and pk.b_cat.shape == (64, 64)
    assert torch.equal(pk.a_cat[:4], ads["b"].down) and torch.equal(pk.a_cat[4:12], ads["a"].down)
    assert torch.all(pk.a_cat[12:] == 0) and torch.all(pk.b_cat[:, 12:] == 0)
    # 12 rank columns in use -> the kernels are promised zeros from column 16 on
    assert pk.r_used == 16 and torch.all(pk.a_cat[pk.r_used:] == 0) and torch.all(pk.b_cat[:, pk.r_used:] == 0)
    assert torch.allclose(pk.col_scale[:4], torch.tensor(2.0 * 1.0 * 0.5))          # alpha = rank
    assert torch.allclose(pk.col_scale[4:12], torch.tensor(0.5 * 16.0 / 8 * 0.5))   # weight * alpha / rank * scale
    # the packed product equals the sum over adapters
    x = torch.randn(5, 16, generator=g)
    got = ((x @ pk.a_cat.T) * pk.col_scale) @ pk.b_cat.T
    ref = sum(ad.multiplier(0.5) * (x @ ad.down.T) @ ad.up.T for ad in ads.values())
    assert torch.allclose(got, ref, atol=1e-5)
    ads["a"].weight = 0.0
    rescale_(pk, ads, 1.0)
    assert torch.all(pk.col_scale[4:12] == 0) and torch.allclose(pk.col_scale[:4], torch.tensor(2.0))
    # GEGLU interleave: blocks of 32 value rows then their 32 gate rows
    t = torch.arange(128).float()[:, None].repeat(1, 2)
    it = interleave_geglu_rows(t)
    assert it[:32, 0].tolist() == list(range(32)) and it[32:64, 0].tolist() == list(range(64, 96))
    assert it[64:96, 0].tolist() == list(range(32, 64)) and it[96:, 0].tolist() == list(range(96, 128))


def test_upstream_state_dict_names_are_remapped():
    import katz_amd.layers as L
    from katz_amd.unet_2d_condition import UNet2DConditionModel, UNetConfig

    L.SKIP_INIT = True
    try:
        unet = UNet2DConditionModel(UNetConfig.tiny())
    finally:
        L.SKIP_INIT = False
    sd = {k: torch.randn_like(v) for k, v in unet.state_dict().items()}
    up = {}
    for k, v in sd.items():
        k2 = k.replace("conv_norm_silu.0.", "conv_norm_out.").replace(".norm_silu1.0.", ".norm1.").replace(".norm_silu2.0.", ".norm2.")
        if ".ff.net.0.proj." in k2:  # the fork's fused-GEGLU split
            h = v.shape[0] // 2
            up[k2.replace(".proj.", ".proj_1.")] = v[:h].clone()
            up[k2.replace(".proj.", ".proj_2.")] = v[h:].clone()
        else:
            up[k2] = v
    unet.load_state_dict(up, strict=True)
    for k, v in unet.state_dict().items():
        assert torch.equal(v, sd[k]), k


def test_euler_schedule_matches_oracle():
    """The product's host-side schedule (numpy) equals the oracle's (torch, KAT-pinned) bit for bit."""
    import torch
    from katz_amd.scheduler import EulerDiscreteScheduler
    from oracle.euler import EulerDiscreteScheduler as OSched

    for cfg, steps in ((dict(beta_start=0.00085, beta_end=0.012, beta_schedule="scaled_linear", timestep_spacing="leading", steps_offset=1), 50),
                       (dict(num_train_timesteps=1100, beta_start=0.0001, beta_end=0.02, beta_schedule="linear"), 10),
                       (dict(beta_schedule="scaled_linear", timestep_spacing="trailing"), 30)):
        p, o = EulerDiscreteScheduler(**cfg), OSched(**cfg)
        assert torch.equal(p.sigmas, o.sigmas)
        assert p.init_noise_sigma.item() == o.init_noise_sigma.item()
        p.set_timesteps(steps)
        o.set_timesteps(steps)
        assert torch.equal(p.timesteps, o.timesteps)
        assert torch.allclose(p.sigmas, o.sigmas, rtol=1e-6, atol=0)
        t = p.coef_table("cpu")
        assert t.shape == (steps, 4) and torch.equal(t[:, 0], p.sigmas[:-1]) and torch.equal(t[:, 1], p.sigmas[1:])
        # unfused step == oracle step on fp32 tensors
        g = torch.Generator().manual_seed(0)
        x, eps = torch.randn(1, 4, 8, 8, generator=g), torch.randn(1, 4, 8, 8, generator=g)
        tt = p.timesteps[0]
        assert torch.equal(p.scale_model_input(x, tt), o.scale_model_input(x, tt))
        assert torch.allclose(p.step(eps, tt, x)[0], o.step(eps, tt, x), rtol=1e-6, atol=1e-6)


def test_expand_lora_scales_docstring_example_and_set_adapters():
    """The worked example in the reference's docstring (unet_loader_utils.py:77-100) is the golden vector."""
    import pytest
    from katz_amd.lora import expand_lora_scales_for_one_adapter as expand, module_weight
    import katz_amd.layers as L
    from katz_amd.unet_2d_condition import UNet2DConditionModel, UNetConfig

    got = expand({"down": 2, "mid": 3, "up": {"block_0": 4, "block_1": [5, 6, 7]}},
                 {"down": [1, 2], "up": [0, 1]}, {"down": 2, "up": 3})
    want = {"down.block_1.0": 2, "down.block_1.1": 2, "down.block_2.0": 2, "down.block_2.1": 2, "mid": 3,
            "up.block_0.0": 4, "up.block_0.1": 4, "up.block_0.2": 4, "up.block_1.0": 5, "up.block_1.1": 6, "up.block_1.2": 7}
    tr = lambda n: "mid_block.attentions.0" if n == "mid" else "{}_blocks.{}.attentions.{}".format(*[p.replace("block_", "") for p in n.split(".")])
    assert got == {tr(k): v for k, v in want.items()}
    assert expand(0.7, {"down": [1], "up": [0]}, {"down": 2, "up": 3}) == 0.7
    assert module_weight(got, "up_blocks.1.attentions.2.transformer_blocks.0.attn1.to_q") == 7.0
    with pytest.raises(RuntimeError):
        module_weight(got, "down_blocks.0.resnets.0.conv1")
    with pytest.raises(ValueError):
        expand({"down": 1.0}, {"down": [1, 2], "up": [0, 1]}, {"down": 2, "up": 3}, ["down_blocks.1.attentions.0.x"])

    L.SKIP_INIT = True
    try:
        unet = UNet2DConditionModel(UNetConfig.tiny())
    finally:
        L.SKIP_INIT = False
    import torch
    for name, m in unet.lora_linears().items():
        m.add_adapter("a", torch.zeros(4, m.in_features), torch.zeros(m.out_features, 4), None)
    unet.set_adapters(["a"], [{"down": 0.5, "mid": 0.25, "up": {"block_0": [0.1, 0.2, 0.3], "block_1": 1.0}}])
    lin = unet.lora_linears()
    w = lambda n: lin[n].adapters["a"].weight
    assert w("down_blocks.1.attentions.1.transformer_blocks.0.attn1.to_q") == 0.5
    assert w("mid_block.attentions.0.proj_in") == 0.25
    assert w("up_blocks.0.attentions.2.transformer_blocks.0.ff.net.2") == 0.3
    assert w("up_blocks.1.attentions.0.transformer_blocks.0.attn2.to_k") == 1.0


def test_shm_adapter_segments_roundtrip():
    """Loader side publishes an adapter into Katz's shared-memory layout; the pipeline side reads it back
    zero-copy (names "<key>_<loader id>", float16, int8 flag array with states 0 / 1 / 10)."""
    import json
    import os
    import pytest
    import torch
    from multiprocessing import shared_memory
    from katz_amd.shm_adapters import ShmAdapterSegments, LOADED

    golden = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "sdxl_lora_keys.json")))
    info = {}
    for wkey in list(golden)[:6]:   # metadata in the reference's schema: {lora key: {"shape", "nbytes"}}
        e = golden[wkey]
        for k, shp in ((e["down_key"], e["down"]), (e["up_key"], e["up"])):
            info[k] = {"shape": shp, "nbytes": shp[0] * shp[1] * 2}
    prefix = f"katztest{os.getpid()}_"
    with pytest.raises(FileNotFoundError):
        ShmAdapterSegments(info, loader_id=0, create=False, name_prefix=prefix)
    loader = ShmAdapterSegments(info, loader_id=0, n_loaders=2, create=True, name_prefix=prefix)
    try:
        reader = ShmAdapterSegments(info, loader_id=0, n_loaders=2, create=False, name_prefix=prefix)
        assert not reader.loaded()
        with pytest.raises(RuntimeError):
            reader.state_dict()
        reader.request(1)
        assert int(loader.flags[0]) == 1
        g = torch.Generator().manual_seed(0)
        sd = {k: torch.randn(*m["shape"], generator=g).to(torch.float16) for k, m in info.items()}
        loader.publish(sd)
        assert reader.loaded() and int(reader.flags[0]) == LOADED
        got = reader.state_dict()
        assert set(got) == set(sd) and all(torch.equal(got[k], sd[k]) and got[k].dtype == torch.float16 for k in sd)
        # the segment of a key is addressable by the reference's name
        k0 = next(iter(info))
        seg = shared_memory.SharedMemory(name=f"{prefix}{k0}_0")
        assert seg.size >= info[k0]["nbytes"]
        seg.close()
        reader.clear()
        assert all(float(a.sum()) == 0 for a in loader.arrays.values())
        del got
        reader.close()
    finally:
        loader.close()


def test_kohya_conversion_reproduces_the_reference_key_list():
    """Kohya / SGM-named keys built by the inverse block arithmetic convert to exactly the 1444 tensor keys (and the
    alpha naming) the reference holds for its converted adapter (tests/golden/sdxl_lora_keys.json, from
    lora_info_shm/TheLastBen_Papercut_SDXL*.json), and load into the UNet."""
    import json
    import os
    import re
    import pytest
    import torch
    from katz_amd.lora_conversion import convert_kohya_lora_to_diffusers

    golden = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "sdxl_lora_keys.json")))

    def kohya_name(mod):  # diffusers module path -> sd-scripts name with SGM block numbering (layers_per_block = 2)
        m = re.match(r"(down_blocks|up_blocks)\.(\d+)\.attentions\.(\d+)\.(.+)", mod)
        if m:
            b, l = int(m.group(2)), int(m.group(3))
            head = f"input_blocks_{b * 3 + l + 1}_1" if m.group(1) == "down_blocks" else f"output_blocks_{b * 3 + l}_1"
            rest = m.group(4)
        else:
            m = re.match(r"mid_block\.attentions\.0\.(.+)", mod)
            head, rest = "middle_block_1", m.group(1)
        return "lora_unet_" + head + "_" + rest.replace(".", "_")

    sd, expect_keys, expect_alpha = {}, set(), {}
    for wkey, e in golden.items():
        mod = wkey[:-len(".weight")]
        kn = kohya_name(mod)
        sd[kn + ".lora_down.weight"] = torch.zeros(e["down"])
        sd[kn + ".lora_up.weight"] = torch.zeros(e["up"])
        sd[kn + ".alpha"] = torch.tensor(e["alpha"])
        expect_keys |= {e["down_key"], e["up_key"]}
        expect_alpha[e["down_key"] + ".alpha" if ".processor." in e["down_key"] else "unet." + mod + ".alpha"] = e["alpha"]
    sd["lora_te1_text_model_encoder_layers_0_mlp_fc1.lora_down.weight"] = torch.zeros(4, 8)
    unet_sd, alphas, rest = convert_kohya_lora_to_diffusers(sd)
    assert len(expect_keys) == 1444 and set(unet_sd) == expect_keys
    assert alphas == expect_alpha and len(alphas) == 722
    assert list(rest) == ["lora_te1_text_model_encoder_layers_0_mlp_fc1.lora_down.weight"]
    for wkey, e in list(golden.items())[:20]:
        assert list(unet_sd[e["down_key"]].shape) == e["down"] and list(unet_sd[e["up_key"]].shape) == e["up"]
    # diffusers-style block names are accepted too; conv targets are refused
    u2, a2, _ = convert_kohya_lora_to_diffusers({
        "lora_unet_down_blocks_1_attentions_0_transformer_blocks_0_attn2_to_out_0.lora_down.weight": torch.zeros(4, 640),
        "lora_unet_down_blocks_1_attentions_0_transformer_blocks_0_attn2_to_out_0.lora_up.weight": torch.zeros(640, 4)})
    assert set(u2) == {"unet.down_blocks.1.attentions.0.transformer_blocks.0.attn2.processor.to_out_lora.down.weight",
                       "unet.down_blocks.1.attentions.0.transformer_blocks.0.attn2.processor.to_out_lora.up.weight"}
    # convolution targets: the renames of lora_conversion_utils.py:78-118 (block numbering) and :178-186 (layer names)
    conv_names = {"input_blocks_4_0_in_layers_2": "down_blocks.1.resnets.0.conv1",
                  "input_blocks_5_0_out_layers_3": "down_blocks.1.resnets.1.conv2",
                  "input_blocks_4_0_skip_connection": "down_blocks.1.resnets.0.conv_shortcut",
                  "input_blocks_3_0_op": "down_blocks.0.downsamplers.0.conv",
                  "output_blocks_2_2_conv": "up_blocks.0.upsamplers.0.conv",
                  "output_blocks_5_0_skip_connection": "up_blocks.1.resnets.2.conv_shortcut",
                  "middle_block_0_in_layers_2": "mid_block.resnets.0.conv1",
                  "middle_block_2_out_layers_3": "mid_block.resnets.1.conv2"}
    csd = {}
    for kn in conv_names:
        csd[f"lora_unet_{kn}.lora_down.weight"] = torch.zeros(4, 4)
        csd[f"lora_unet_{kn}.lora_up.weight"] = torch.zeros(4, 4)
    u3, _, _ = convert_kohya_lora_to_diffusers(csd)
    assert set(u3) == {f"unet.{v}.lora.{w}.weight" for v in conv_names.values() for w in ("down", "up")}
    with pytest.raises(NotImplementedError):   # a resnet's time_emb_proj carries no LoRA here
        convert_kohya_lora_to_diffusers({"lora_unet_input_blocks_4_0_emb_layers_1.lora_down.weight": torch.zeros(4, 4)})
    with pytest.raises(ValueError):
        convert_kohya_lora_to_diffusers({"lora_unet_middle_block_1_proj_in.lora_down.weight": torch.zeros(4, 4)})

    # end to end on the SDXL-shaped module tree: every converted key finds its LoRALinear
    import katz_amd.layers as L
    from katz_amd.unet_2d_condition import UNet2DConditionModel, UNetConfig
    L.SKIP_INIT = True
    try:
        unet = UNet2DConditionModel(UNetConfig.sdxl())
    finally:
        L.SKIP_INIT = False
    unet.load_lora_into_unet(unet_sd, network_alphas=alphas, adapter_name="papercut")
    lin = unet.lora_linears()
    assert sum("papercut" in m.adapters for m in lin.values()) == 722
    m = lin["down_blocks.1.attentions.0.transformer_blocks.0.attn1.to_q"]
    assert m.adapters["papercut"].alpha == 20000.0


def test_unet_lora_surface_reaches_convolutions():
    """Adapters that target convolutions (diffusers key spelling; 3x3 and the 1x1 conv_shortcut) register on the
    Conv3x3 / Conv1x1 modules and follow set_adapters / fuse_lora / delete_adapters like the linear ones."""
    import pytest
    import torch
    import katz_amd.layers as L
    from katz_amd.unet_2d_condition import UNet2DConditionModel, UNetConfig

    torch.manual_seed(0)
    unet = UNet2DConditionModel(UNetConfig.tiny())     # initialised weights: fuse checks the merged weights are finite
    convs = unet.lora_convs()
    assert "down_blocks.0.resnets.0.conv1" in convs and "down_blocks.0.downsamplers.0.conv" in convs
    assert "conv_in" in convs and "down_blocks.1.resnets.0.conv_shortcut" in convs
    c = convs["down_blocks.0.resnets.0.conv1"]
    lin_name = "down_blocks.1.attentions.0.transformer_blocks.0.attn1.to_q"
    lin = unet.lora_linears()[lin_name]
    sd = {"unet.down_blocks.0.resnets.0.conv1.lora.down.weight": torch.zeros(4, c.in_channels, 3, 3),
          "unet.down_blocks.0.resnets.0.conv1.lora.up.weight": torch.zeros(c.out_channels, 4, 1, 1),
          f"unet.{lin_name}.lora.down.weight": torch.zeros(4, lin.in_features),
          f"unet.{lin_name}.lora.up.weight": torch.zeros(lin.out_features, 4)}
    unet.load_lora_into_unet(sd, network_alphas={"unet.down_blocks.0.resnets.0.conv1.alpha": 8.0}, adapter_name="locon")
    assert c.adapters["locon"].alpha == 8.0 and c.active == ["locon"] and lin.active == ["locon"]
    unet.set_adapters(["locon"], [0.5])
    assert c.adapters["locon"].weight == 0.5 and c.adapters["locon"].multiplier() == 0.5 * 8.0 / 4
    unet.set_adapters(["locon"], [{"down": 0.3}])      # block dictionaries address transformers; the conv keeps 1.0
    assert lin.adapters["locon"].weight == 0.3 and c.adapters["locon"].weight == 1.0
    # the 1x1 shortcut takes [r,Cin,1,1] / [Cout,r,1,1] (LoRAConv2dLayer, models/lora.py:258-296); wrong shapes are refused
    sc = convs["down_blocks.1.resnets.0.conv_shortcut"]
    g = torch.Generator().manual_seed(0)
    unet.load_lora_into_unet({"unet.down_blocks.1.resnets.0.conv_shortcut.lora.down.weight": torch.randn(4, 64, 1, 1, generator=g),
                              "unet.down_blocks.1.resnets.0.conv_shortcut.lora.up.weight": torch.randn(128, 4, 1, 1, generator=g)},
                             adapter_name="short")
    assert sc.active == ["short"] and sc.adapters["short"].down.shape == (4, 64)
    with pytest.raises(ValueError):
        unet.load_lora_into_unet({"unet.down_blocks.1.resnets.0.conv_shortcut.lora.down.weight": torch.zeros(4, 32, 1, 1),
                                  "unet.down_blocks.1.resnets.0.conv_shortcut.lora.up.weight": torch.zeros(128, 4, 1, 1)},
                                 adapter_name="bad")
    # fusing merges conv adapters through the merged-kernel identity (models/lora.py:403-421) and unfusing restores
    with torch.no_grad():
        c.adapters["locon"].down.copy_(torch.randn(c.adapters["locon"].down.shape, generator=g) * 0.1)
        c.adapters["locon"].up.copy_(torch.randn(c.adapters["locon"].up.shape, generator=g) * 0.1)
    unet.set_adapters(["locon", "short"], [0.5, 2.0])
    w_c, w_sc = c.weight.detach().clone(), sc.weight.detach().clone()
    unet.fuse_lora(lora_scale=0.7)
    ad = c.adapters["locon"]
    want = w_c + 0.7 * 0.5 * 8.0 / 4 * (ad.up.reshape(c.out_channels, -1) @ ad.down.reshape(4, -1)).reshape(w_c.shape)
    assert torch.allclose(c.weight, want, atol=1e-5) and c._fused == {"locon": 0.7 * 0.5 * 8.0 / 4}
    ads = sc.adapters["short"]
    want = w_sc + 0.7 * 2.0 * (ads.up @ ads.down).reshape(w_sc.shape)
    assert torch.allclose(sc.weight, want, atol=1e-5)
    assert c._lora_pack() == (None, None) and sc._pack() is None       # fused adapters are not applied a second time
    unet.unfuse_lora()
    assert torch.allclose(c.weight, w_c, atol=1e-5) and torch.allclose(sc.weight, w_sc, atol=1e-5) and not c._fused
    unet.delete_adapters(["locon", "short"])
    assert not c.adapters and not lin.adapters and not sc.adapters


def test_fuse_that_fails_leaves_everything_as_it_was():
    """A non-finite merged weight raises (the reference's safe_fusing, models/lora.py:416-421) and neither the layer
    that failed nor the layers merged before it keep any trace: weights bit for bit, no adapter marked as fused."""
    import pytest
    import torch
    import katz_amd.layers as L
    from katz_amd.unet_2d_condition import UNet2DConditionModel, UNetConfig

    torch.manual_seed(0)
    unet = UNet2DConditionModel(UNetConfig.tiny())
    lin = unet.lora_linears()
    g = torch.Generator().manual_seed(1)
    names = list(lin)
    for n in names:
        m = lin[n]
        m.add_adapter("a", torch.randn(4, m.in_features, generator=g) * 0.1, torch.randn(m.out_features, 4, generator=g) * 0.1)
    bad = names[len(names) // 2]
    lin[bad].adapters["a"].up[0, 0] = float("inf")
    for m in lin.values():
        m.active = ["a"]
    before = {n: lin[n].weight.detach().clone() for n in names}
    with pytest.raises(ValueError):
        unet.fuse_lora()
    for n in names:
        assert torch.equal(lin[n].weight, before[n]), n
        assert not lin[n]._fused, n
    # one layer on its own: same guarantee
    with pytest.raises(ValueError):
        lin[bad].fuse()
    assert torch.equal(lin[bad].weight, before[bad]) and not lin[bad]._fused
    # and with the bad adapter repaired the whole model fuses and unfuses
    lin[bad].adapters["a"].up[0, 0] = 0.0
    unet.fuse_lora()
    assert all(m._fused for m in lin.values())
    unet.unfuse_lora()
    assert max((lin[n].weight - before[n]).abs().max().item() for n in names) < 1e-5


def test_pack_adapters_cuts_wide_rank_sums_into_packs_of_128():
    """Sum of active ranks above 128 (three rank-64 adapters; one rank-200 adapter): the rank rows are cut, in order,
    into packs of at most 128 columns; every pack reproduces its slice of sum_i s_i B_i A_i; rescaling reaches all."""
    import torch
    from katz_amd.lora import Adapter, pack_adapters, rescale_

    g = torch.Generator().manual_seed(0)
    K, N = 48, 40
    for ranks in ([64, 64, 64], [200], [100, 30, 7]):
        ads = {f"a{i}": Adapter(torch.randn(r, K, generator=g), torch.randn(N, r, generator=g), alpha=2.0 * r, weight=0.5 + i)
               for i, r in enumerate(ranks)}
        p = pack_adapters(ads, list(ads), K, N, torch.float32, "cpu", 1.0)
        packs = [p, *p.overflow]
        assert all(q.R <= 128 and q.R % 64 == 0 for q in packs)
        assert sum(r for q in packs for _, _, r in q.spans) == sum(ranks)
        delta = sum((q.b_cat * q.col_scale) @ q.a_cat for q in packs)
        want = sum(a.multiplier() * (a.up @ a.down) for a in ads.values())
        assert torch.allclose(delta, want, atol=1e-3)
        for a in ads.values():
            a.weight *= 2
        rescale_(p, ads, 0.5)
        delta = sum((q.b_cat * q.col_scale) @ q.a_cat for q in packs)
        assert torch.allclose(delta, want, atol=1e-3)       # weights doubled, global scale halved
    assert len(pack_adapters({"a": Adapter(torch.zeros(96, K), torch.zeros(N, 96))}, ["a"], K, N, torch.float32, "cpu").overflow) == 0


def test_bench_refuses_more_than_one_gpu():
    """bench.py --gpus N with N > 1 exits with a message: this build runs on one GPU (no collectives, no sharding)."""
    import subprocess
    import sys
    from pathlib import Path

    root = Path(__file__).resolve().parent.parent
    r = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2 and "ONE GPU" in r.stderr


def _fake_prefetch_lib(monkeypatch, calls):
    from katz_amd import ops

    class FakeLib:
        def kh_set_weight_prefetch(self, ptr, nbytes):
            calls.append((ptr, nbytes))
            return 0

    monkeypatch.setattr(ops._lib, "load", lambda: FakeLib())
    monkeypatch.setattr(ops._lib, "is_loaded", lambda: True)
    monkeypatch.setattr(ops, "WEIGHT_PREFETCH", True)


def test_weight_prefetch_hints_are_learned_from_the_previous_pass(monkeypatch):
    """ops._weight_prefetch_hint inside one model's scope: the first pass over a sequence of launches gives no hints; the
    second hints, at launch i, the operands of launch i + 1 - weights only for long rows (K >= 2560 or a 3x3 kernel) or
    below the size limit, adapter matrices always; a tensor that has been freed is dropped instead of hinted."""
    import gc

    from katz_amd import ops

    calls = []
    _fake_prefetch_lib(monkeypatch, calls)
    monkeypatch.setattr(ops, "PREFETCH_SMALL_BYTES", 16 << 10)
    model = torch.nn.Identity()
    w_small = torch.zeros(8, 1280)             # K 1280 and 40 KB, above the size limit set here: not hinted
    w_long = torch.zeros(8, 5120)              # K 5120: hinted
    w_conv = torch.zeros(4, 3, 3, 320)         # 9 * 320 = 2880: hinted
    a_cat, b_cat = torch.zeros(128, 5120), torch.zeros(8, 128)
    seq = [(w_small, None, None), (w_long, a_cat, b_cat), (w_conv, None, None)]
    hinted = lambda: [c for c in calls if c[0] is not None]
    with ops.weight_prefetch_scope(model) as table:
        for w, a, b in seq:
            ops._weight_prefetch_hint(w, a, b)
    assert hinted() == []                       # nothing known on the first pass
    with ops.weight_prefetch_scope(model) as table2:
        assert table2 is table                  # the same model: the same table
        for w, a, b in seq:
            ops._weight_prefetch_hint(w, a, b)
    assert hinted() == [(w_long.data_ptr(), w_long.numel() * 4), (a_cat.data_ptr(), a_cat.numel() * 4),
                        (b_cat.data_ptr(), b_cat.numel() * 4), (w_conv.data_ptr(), w_conv.numel() * 4)]
    # a forward starts without a predecessor: the last launch of a pass learns nothing about the next pass's first
    assert w_conv.data_ptr() not in table and set(table) == {w_small.data_ptr(), w_long.data_ptr()}
    # the size limit admits small weights whatever their K (the default admits the d x d layers)
    monkeypatch.setattr(ops, "PREFETCH_SMALL_BYTES", 64 << 10)
    calls.clear()
    with ops.weight_prefetch_scope(model):
        ops._weight_prefetch_hint(w_conv)
        ops._weight_prefetch_hint(w_small)      # learned: w_small follows w_conv
    calls.clear()
    with ops.weight_prefetch_scope(model):
        ops._weight_prefetch_hint(w_conv)
    assert hinted() == [(w_small.data_ptr(), w_small.numel() * 4)]
    # a freed successor: dropped
    key = w_small.data_ptr()
    del w_long, seq, w, a, b
    gc.collect()
    calls.clear()
    with ops.weight_prefetch_scope(model):
        ops._weight_prefetch_hint(w_small)
    assert hinted() == [] and key not in table


def test_weight_prefetch_hints_never_cross_models_or_forwards(monkeypatch):
    """A hinted pointer is baked into a captured graph, so it must belong to the model whose forward issues it: every
    model learns into a table of its own, a launch outside any model's forward neither learns nor hints, whatever is
    still pending in the library is cleared before every new hint and at the end of a scope, and a model that is freed
    takes its table with it."""
    import gc

    from katz_amd import ops

    calls = []
    _fake_prefetch_lib(monkeypatch, calls)
    monkeypatch.setattr(ops, "PREFETCH_SMALL_BYTES", 1 << 30)
    unet, cnet = torch.nn.Identity(), torch.nn.Identity()
    wu = [torch.zeros(8, 64) for _ in range(3)]
    wc = [torch.zeros(8, 64) for _ in range(2)]
    stray = torch.zeros(8, 64)
    hinted = lambda: [c[0] for c in calls if c[0] is not None]

    def loop():                     # ControlNet -> UNet -> a stand-alone launch, as an eager denoise loop issues them
        with ops.weight_prefetch_scope(cnet):
            for w in wc:
                ops._weight_prefetch_hint(w)
        with ops.weight_prefetch_scope(unet):
            for w in wu:
                ops._weight_prefetch_hint(w)
        ops._weight_prefetch_hint(stray)

    loop()
    assert hinted() == []
    calls.clear()
    loop()
    # inside the ControlNet only its own second weight is hinted, inside the UNet only its own second and third:
    # nothing of the other model, nothing of the stand-alone launch, and the last launch of a model hints nothing
    assert hinted() == [wc[1].data_ptr(), wu[1].data_ptr(), wu[2].data_ptr()]
    tu, tc = ops._pf_tables[unet], ops._pf_tables[cnet]
    assert set(tu) == {wu[0].data_ptr(), wu[1].data_ptr()} and set(tc) == {wc[0].data_ptr()}
    assert ops._pf_next[0] is None and ops._pf_last[0] is None
    # every hint call first clears what may be pending (a launch that was refused never consumed its hint) ...
    calls.clear()
    ops._weight_prefetch_hint(stray)
    assert calls == [(None, 0)]
    # ... and so does the end of a scope
    calls.clear()
    with ops.weight_prefetch_scope(unet):
        ops._weight_prefetch_hint(wu[0])
    assert calls[-1] == (None, 0) and hinted() == [wu[1].data_ptr()]
    # a freed model: its table goes with it
    n = len(ops._pf_tables)
    del cnet, tc
    gc.collect()
    assert len(ops._pf_tables) == n - 1
