"""conv1 of a residual block that leaves the statistics of the GroupNorm (+ SiLU) behind it as a by-product of its epilogue
(kh_conv3x3_gn_stats_nhwc_bf16, then kh_group_norm_apply_bf16) against the oracle's GroupNorm of torch's fp32 convolution
(rounded to bf16 where the reference's half-precision modules round: the convolution's result, the time-embedding term)
and against the library's own convolution followed by kh_group_norm_bf16.

Tolerance: the parity contract's 2e-2 * (|ref| + rms(ref)) for bf16 kernels against the oracle; against the library's
two-kernel form the statistics differ by summation order only (fp32 partial sums per tile against per pixel range):
identical up to the last bf16 digit (1e-2 of the same bound) of a few elements (fewer than 2 %).
"""
import pytest
import torch

from helpers import assert_close_rel, bf16_round
from oracle import ops as O

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def dev():
    return torch.device("cuda:0")


def randn(g, *shape, std=1.0):
    return bf16_round(torch.randn(*shape, generator=g) * std)


def say(*a):
    print(*a, flush=True)


def _case(Nb, Cin, Cout, H, seed):
    g = torch.Generator().manual_seed(seed)
    x = randn(g, Nb, Cin, H, H)
    w = randn(g, Cout, Cin, 3, 3, std=(9 * Cin) ** -0.5)
    b = randn(g, Cout, std=0.3)
    gamma = bf16_round(1.0 + 0.3 * torch.randn(Cout, generator=g))
    beta = randn(g, Cout, std=0.3)
    add = randn(g, Nb, Cout, std=0.5)
    return x, w, b, gamma, beta, add


def _ref(x, w, b, gamma, beta, add, G, eps, act):
    y = bf16_round(torch.nn.functional.conv2d(x, w, b, padding=1))       # the convolution's bf16 result
    if add is not None:
        y = y + add[:, :, None, None]
    return O.group_norm(y, G, gamma, beta, eps, act)


@pytest.mark.parametrize("Nb,Cin,Cout,H,act,with_add", [
    (2, 320, 320, 128, "silu", True),      # SDXL's 128x128 level: 128x160 tiles, 128 row tiles per image, 10-channel groups
    (2, 1280, 1280, 32, "silu", True),     # 32x32 level: 64x160 tiles, 16 row tiles per image, 40-channel groups
    (2, 2560, 1280, 32, "silu", True),     # first resnet of the first up block
    (2, 640, 640, 64, "silu", True),       # 64x64 level: 128x160 tiles, 32 row tiles per image, 20-channel groups
    (2, 320, 640, 64, "silu", True),       # first resnet of the second down block
    (2, 1920, 640, 64, "none", False),     # no activation, no time-embedding term
    (1, 640, 640, 64, "silu", True),       # one image: 64x160 tiles, 64 row tiles
])
def test_convolution_that_leaves_the_norm_statistics(Nb, Cin, Cout, H, act, with_add):
    from katz_amd import ops
    say("conv3x3 + group norm", Nb, Cin, Cout, H, act, with_add)
    d = dev()
    G, eps = 32, 1e-5
    x, w, b, gamma, beta, add = _case(Nb, Cin, Cout, H, seed=Cin + Cout + H + Nb)
    if not with_add:
        add = None
    xd = x.to(d, BF).contiguous(memory_format=torch.channels_last)
    splits = ops.conv3x3_gn_splits(xd, Cout, G)
    assert splits in (H * H // 64, H * H // 128), splits   # 64- or 128-row tiles, whichever the convolution runs on
    wp = ops.pack_conv3x3_weight(w.to(d, BF))
    args = (b.to(d, BF), G, gamma.to(d, BF), beta.to(d, BF), eps, act)
    addd = None if add is None else add.to(d, BF)
    y = ops.conv3x3_group_norm(xd, wp, *args, add_nc=addd)
    y_again = ops.conv3x3_group_norm(xd, wp, *args, add_nc=addd)
    # the library's two kernels
    c = ops.conv3x3(xd, wp, b.to(d, BF))
    y2 = ops.group_norm(c, G, gamma.to(d, BF), beta.to(d, BF), eps, act, add_nc=addd)
    torch.cuda.synchronize()
    assert y.shape == (Nb, Cout, H, H) and y.is_contiguous(memory_format=torch.channels_last)
    assert torch.equal(y, y_again), "deterministic: fixed summation orders"
    ref = _ref(x, w, b, gamma, beta, add, G, eps, act)
    assert_close_rel(y, ref, 2e-2, "convolution with statistics + GroupNorm's second pass against the oracle")
    assert_close_rel(y, y2.float().cpu(), 1e-2, "statistics from the convolution against convolution + kh_group_norm_bf16")
    frac = (y != y2).float().mean().item()
    say(f"  elements that differ from the two-kernel form in their last digit: {100 * frac:.3f} %")
    assert frac < 0.02


def test_statistics_against_plain_sums():
    """The partial sums themselves: folded over the row tiles they equal the sums of the convolution's stored result
    (residual included) plus the per-channel term."""
    from katz_amd import ops
    say("conv3x3 statistics against torch sums")
    d = dev()
    Nb, Cin, Cout, H, G = 2, 640, 640, 64, 32
    x, w, b, _, _, add = _case(Nb, Cin, Cout, H, seed=3)
    g = torch.Generator().manual_seed(4)
    res = randn(g, Nb, Cout, H, H).to(d, BF).contiguous(memory_format=torch.channels_last)
    xd = x.to(d, BF).contiguous(memory_format=torch.channels_last)
    wp = ops.pack_conv3x3_weight(w.to(d, BF))
    addd = add.to(d, BF)
    for residual, add_nc in ((None, addd), (res, None), (res, addd)):
        conv, part, splits = ops.conv3x3_stats(xd, wp, b.to(d, BF), G, add_nc=add_nc, residual=residual)
        torch.cuda.synchronize()
        assert torch.equal(conv, ops.conv3x3(xd, wp, b.to(d, BF), residual=residual)), "the convolution's own result is untouched"
        assert part.shape == (Nb, G, splits, 2) and torch.isfinite(part).all(), "every (image, group, row tile) slot is written"
        v = conv.float() if add_nc is None else conv.float() + add_nc.float()[:, :, None, None]
        v = v.double().reshape(Nb, G, Cout // G, H * H)
        s_ref, q_ref = v.sum(dim=(2, 3)), (v * v).sum(dim=(2, 3))
        got = part.double().sum(dim=2)
        assert torch.allclose(got[..., 0], s_ref, rtol=1e-4, atol=2e-2), "sums"
        assert torch.allclose(got[..., 1], q_ref, rtol=1e-4), "sums of squares"


@pytest.mark.parametrize("act", ["none", "silu"])
def test_norm_behind_a_convolution_with_residual(act):
    """conv2 + skip, then the next module's GroupNorm (no per-channel term) on the statistics conv2 left."""
    from katz_amd import ops
    say("conv3x3 + residual, statistics, group norm", act)
    d = dev()
    Nb, Cin, Cout, H, G, eps = 2, 1280, 1280, 32, 32, 1e-6
    x, w, b, gamma, beta, _ = _case(Nb, Cin, Cout, H, seed=9)
    g = torch.Generator().manual_seed(10)
    res = randn(g, Nb, Cout, H, H)
    xd = x.to(d, BF).contiguous(memory_format=torch.channels_last)
    resd = res.to(d, BF).contiguous(memory_format=torch.channels_last)
    wp = ops.pack_conv3x3_weight(w.to(d, BF))
    y, part, splits = ops.conv3x3_stats(xd, wp, b.to(d, BF), G, residual=resd)
    n = ops.group_norm_from_stats(y, G, gamma.to(d, BF), beta.to(d, BF), eps, act, part, splits)
    n2 = ops.group_norm(y, G, gamma.to(d, BF), beta.to(d, BF), eps, act)
    torch.cuda.synchronize()
    conv = bf16_round(bf16_round(torch.nn.functional.conv2d(x, w, b, padding=1)) + res)   # rounded, residual added, rounded
    ref = O.group_norm(conv, G, gamma, beta, eps, act)
    assert_close_rel(n, ref, 2e-2, "norm on the convolution's statistics against the oracle")
    assert_close_rel(n, n2.float().cpu(), 1e-2, "against kh_group_norm_bf16 on the same tensor")
    assert (n != n2).float().mean().item() < 0.02


def test_shapes_that_are_not_taken():
    from katz_amd import _lib, ops
    say("conv3x3 + group norm, refused shapes")
    d = dev()
    x2 = torch.zeros((2, 640, 64, 64), dtype=BF, device=d).contiguous(memory_format=torch.channels_last)
    assert ops.conv3x3_gn_splits(x2, 640, 32) == 32
    assert ops.conv3x3_gn_splits(x2, 640, 10) == 0         # 64-channel groups do not divide the 160-column tiles
    assert ops.conv3x3_gn_splits(x2, 648, 8) == 0          # output width not a multiple of 160
    assert ops.conv3x3_gn_splits(x2, 640, 32, stride=2) == 16   # a stride-2 convolution: 32x32 outputs on 64-row tiles
    x3 = torch.zeros((2, 640, 60, 60), dtype=BF, device=d).contiguous(memory_format=torch.channels_last)
    assert ops.conv3x3_gn_splits(x3, 640, 32) == 0         # 3600 pixels per image: no whole number of 128-row tiles
    x4 = torch.zeros((2, 64, 16, 16), dtype=BF, device=d).contiguous(memory_format=torch.channels_last)
    assert ops.conv3x3_gn_splits(x4, 160, 32) == 0         # a small convolution runs on the 128 x 128 tiles
    w = torch.zeros((160, 3, 3, 64), dtype=BF, device=d)
    with pytest.raises(_lib.KatzHipError):
        ops.conv3x3_group_norm(x4, w, None, 32, None, None)


@pytest.mark.parametrize("cin,cout,H", [(1280, 1280, 32), (320, 640, 64), (320, 320, 128)])
def test_resnet_block_with_and_without_the_norm_in_the_convolution(monkeypatch, cin, cout, H):
    """ResnetBlock2D at SDXL's widths: norm2 on the statistics conv1 leaves against the same module running convolution
    and norm one after the other, and both against the oracle's block."""
    import katz_amd.layers as L
    from helpers import cosine, round_module_to_bf16_
    from katz_amd import ops
    from oracle import blocks as OB

    say("resnet block, norm2 statistics from conv1 on / off", cin, cout, H)
    d = dev()
    torch.manual_seed(5)
    oracle = OB.ResnetBlock2D(in_channels=cin, out_channels=cout, temb_channels=1280, eps=1e-5)
    for m in oracle.modules():
        if isinstance(m, torch.nn.GroupNorm) or hasattr(m, "num_groups"):
            if getattr(m, "weight", None) is not None:
                torch.nn.init.normal_(m.weight, 1.0, 0.2); torch.nn.init.normal_(m.bias, 0.0, 0.2)
    round_module_to_bf16_(oracle)
    prod = L.ResnetBlock2D(in_channels=cin, out_channels=cout, temb_channels=1280, eps=1e-5)
    prod.load_state_dict(oracle.state_dict(), strict=True)
    prod = prod.to(d, BF)
    g = torch.Generator().manual_seed(6)
    x = bf16_round(torch.randn(2, cin, H, H, generator=g))
    temb = bf16_round(torch.randn(2, 1280, generator=g))
    xd = x.to(d, BF).contiguous(memory_format=torch.channels_last)
    temb_act = torch.nn.functional.silu(temb.to(d, BF))
    with torch.no_grad():
        ref = oracle(x, temb)
        assert L.CONV_GN_FUSE
        ops.CALL_LOG = []
        y1 = prod(xd, temb_act)
        log1, ops.CALL_LOG = ops.CALL_LOG, None
        monkeypatch.setattr(L, "CONV_GN_FUSE", False)
        ops.CALL_LOG = []
        y0 = prod(xd, temb_act)
        log0, ops.CALL_LOG = ops.CALL_LOG, None
    torch.cuda.synchronize()
    assert sum(1 for e in log1 if e[0] == "group_norm_apply") == 1 and sum(1 for e in log1 if e[0] == "group_norm") == 1
    assert sum(1 for e in log0 if e[0] == "group_norm") == 2 and not any(e[0] == "group_norm_apply" for e in log0)
    c1, c0, c10 = cosine(y1, ref), cosine(y0, ref), cosine(y1, y0)
    say(f"  cosine against the oracle: fused {c1:.6f}, separate {c0:.6f}; fused against separate {c10:.6f}")
    assert c1 >= 0.9995 and c0 >= 0.9995 and c10 >= 0.9995
    assert_close_rel(y1, ref, 4e-2, "resnet block with norm2's statistics from conv1")
    assert_close_rel(y1, y0.float().cpu(), 2e-2, "statistics from conv1 against the separate kernels")


def test_statistics_ride_from_one_block_to_the_next(monkeypatch):
    """Two residual blocks in a row: the second block's norm1 runs on what the first block's conv2 left (one full
    GroupNorm in all: the first block's norm1), against the same modules without the hand-over and against the oracle.
    A tensor modified in place after the convolution loses its statistics."""
    import katz_amd.layers as L
    from helpers import cosine, round_module_to_bf16_
    from katz_amd import ops
    from oracle import blocks as OB

    say("two resnet blocks, statistics handed from conv2 to the next norm1")
    d = dev()
    torch.manual_seed(7)
    oracle = torch.nn.ModuleList([OB.ResnetBlock2D(in_channels=640, out_channels=640, temb_channels=1280, eps=1e-5) for _ in range(2)])
    for m in oracle.modules():
        if isinstance(m, torch.nn.GroupNorm):
            torch.nn.init.normal_(m.weight, 1.0, 0.2); torch.nn.init.normal_(m.bias, 0.0, 0.2)
    round_module_to_bf16_(oracle)
    prod = torch.nn.ModuleList([L.ResnetBlock2D(in_channels=640, out_channels=640, temb_channels=1280, eps=1e-5) for _ in range(2)])
    prod.load_state_dict(oracle.state_dict(), strict=True)
    prod = prod.to(d, BF)
    g = torch.Generator().manual_seed(8)
    x = bf16_round(torch.randn(2, 640, 64, 64, generator=g))
    temb = bf16_round(torch.randn(2, 1280, generator=g))
    xd = x.to(d, BF).contiguous(memory_format=torch.channels_last)
    temb_act = torch.nn.functional.silu(temb.to(d, BF))

    def run():
        ops.CALL_LOG = []
        try:
            h = xd
            for blk in prod:
                h = blk(h, temb_act)
        finally:
            log, ops.CALL_LOG = ops.CALL_LOG, None
        return h, log

    with torch.no_grad():
        ref = oracle[1](oracle[0](x, temb), temb)
        y1, log1 = run()
        assert getattr(y1, "_katz_gn_stats", None) is not None, "the last conv2 leaves statistics for whoever follows"
        # an in-place change invalidates them: the norm falls back to its own statistics pass
        y_mod = y1.clone(); y_mod._katz_gn_stats = y1._katz_gn_stats
        ops.residual_add_(y_mod, [torch.ones_like(y_mod)])
        ops.CALL_LOG = []
        n_mod = prod[0].norm_silu1(y_mod)
        log_mod, ops.CALL_LOG = ops.CALL_LOG, None
        n_ref = ops.group_norm(y_mod, 32, prod[0].norm_silu1[0].weight, prod[0].norm_silu1[0].bias, 1e-5, "silu")
        monkeypatch.setattr(L, "CONV_GN_FUSE", False)
        y0, log0 = run()
    torch.cuda.synchronize()
    assert [e[0] for e in log_mod] == ["group_norm"] and torch.equal(n_mod, n_ref)
    assert sum(1 for e in log1 if e[0] == "group_norm") == 1 and sum(1 for e in log1 if e[0] == "group_norm_apply") == 3
    assert sum(1 for e in log0 if e[0] == "group_norm") == 4 and not any(e[0] == "group_norm_apply" for e in log0)
    c1, c0 = cosine(y1, ref), cosine(y0, ref)
    say(f"  cosine against the oracle: with the hand-over {c1:.6f}, without {c0:.6f}")
    assert c1 >= 0.9995 and c0 >= 0.9995
    assert_close_rel(y1, ref, 4e-2, "two blocks with the statistics handed over")
    assert_close_rel(y1, y0.float().cpu(), 2e-2, "hand-over against separate kernels")
