"""Parity of every katz_hip kernel (through the C ABI) against the CPU oracle on seeded inputs.

Tolerances: bf16 kernels -- elementwise |err| <= 2e-2 * (|ref| + rms(ref)) against the oracle evaluated
in fp32 on the same bf16-rounded inputs; fp32 path -- 1e-4; pure data movement / single-rounding adds --
bit exact.
"""
import math

import pytest
import torch

from helpers import cosine, assert_close_rel, bf16_round
from oracle import ops as O

pytestmark = pytest.mark.gpu

BF = torch.bfloat16
REL_BF16 = 2e-2


def dev():
    return torch.device("cuda:0")


def randn(gen, *shape, std=1.0):
    return bf16_round(torch.randn(*shape, generator=gen) * std)


def say(*a):
    print(*a, flush=True)


# ------------------------------------------------------------------------------------------- K1
def _lora_case(M, N, K, ranks, scales, bias=True, residual=False, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = randn(g, M, K)
    w = randn(g, N, K, std=0.02)
    b = randn(g, N, std=0.02) if bias else None
    adapters = []
    for r, s in zip(ranks, scales):
        adapters.append((randn(g, r, K, std=0.02), randn(g, N, r, std=0.02), s))
    res = randn(g, M, N) if residual else None
    return x, w, b, adapters, res


def _run_lora(x, w, b, adapters, res, geglu=False, tile=0):
    from katz_amd import ops
    from katz_amd.lora import Adapter, pack_adapters

    d = dev()
    N, K = w.shape
    ads = {f"a{i}": Adapter(A, B, alpha=None, weight=s) for i, (A, B, s) in enumerate(adapters)}
    packed = pack_adapters(ads, list(ads), K, N, BF, d, geglu_interleave=geglu) if ads else None
    wd, bd = w, b
    if geglu:
        from katz_amd.lora import interleave_geglu_rows
        wd = interleave_geglu_rows(w)
        bd = interleave_geglu_rows(b) if b is not None else None
    y = ops.lora_linear(
        x.to(d, BF), wd.to(d, BF), None if bd is None else bd.to(d, BF),
        None if packed is None else packed.a_cat, None if packed is None else packed.b_cat,
        None if packed is None else packed.col_scale, None if res is None else res.to(d, BF),
        geglu=geglu, tile=tile)
    torch.cuda.synchronize()
    return y


LORA_SHAPES = [
    # M, N, K, ranks, scales, bias, residual
    (2048, 1280, 1280, (64,), (1.0,), False, False),      # to_q at 32x32, one rank-64 adapter
    (8192, 640, 640, (64, 32), (0.8, 0.6), True, True),   # to_out.0 at 64x64, two adapters + residual
    (154, 1280, 2048, (64, 32), (0.8, 0.6), False, False),  # cross-attention to_k / to_v (77 tokens x 2)
    (2048, 1280, 5120, (64, 32), (0.8, 0.6), True, True),   # ff.net.2
    (8192, 640, 640, (), (), True, False),                  # adapter-free
    (100, 136, 72, (8,), (2.0,), True, True),               # ragged: partial tiles in M, N, K and rank padding
    (1, 8, 8, (16, 8, 4), (1.0, 0.5, 0.25), True, False),   # minimum sizes
    (300, 1280, 320, (128,), (1.0,), True, False),          # maximum packed rank
]


@pytest.mark.parametrize("tile", [0, 1, 2])
@pytest.mark.parametrize("case", LORA_SHAPES, ids=lambda c: f"M{c[0]}N{c[1]}K{c[2]}r{'+'.join(map(str, c[3])) or '0'}")
def test_lora_linear_bf16(case, tile):
    M, N, K, ranks, scales, bias, residual = case
    if tile == 2 and (sum(ranks) + 63) // 64 * 64 > 96:
        pytest.skip("256x128 tile of the simple kernel is built for packed rank <= 96")
    say("lora_linear_bf16", case, "tile", tile)
    x, w, b, adapters, res = _lora_case(M, N, K, ranks, scales, bias, residual)
    y = _run_lora(x, w, b, adapters, res, tile=tile)
    ref = O.lora_linear(x, w, b, adapters, res)
    assert_close_rel(y, ref, REL_BF16, "lora_linear_bf16")
    # merge identity: the same result as a plain linear with W + sum s B A
    ref2 = torch.nn.functional.linear(x, O.lora_merged_weight(w, adapters), b)
    if res is not None:
        ref2 = ref2 + res
    assert_close_rel(y, ref2, REL_BF16, "lora_linear_bf16 vs merged weight")


@pytest.mark.parametrize("case", [c for c in LORA_SHAPES if c[3] and c[2] % 64 == 0],
                         ids=lambda c: f"M{c[0]}N{c[1]}K{c[2]}r{'+'.join(map(str, c[3]))}")
def test_lora_shrink_then_pre_gemm(case):
    """Two-launch form: t = shrink(x), y = x W^T + b + t B^T; same oracle, same tolerance."""
    from katz_amd import ops
    from katz_amd.lora import Adapter, pack_adapters

    M, N, K, ranks, scales, bias, residual = case
    say("lora shrink + pre gemm", case)
    x, w, b, adapters, res = _lora_case(M, N, K, ranks, scales, bias, residual)
    d = dev()
    ads = {f"a{i}": Adapter(A, B, alpha=None, weight=s) for i, (A, B, s) in enumerate(adapters)}
    pk = pack_adapters(ads, list(ads), K, N, BF, d)
    xd = x.to(d, BF)
    t = ops.lora_shrink(xd, pk.a_cat, pk.col_scale)
    torch.cuda.synchronize()
    t_ref = torch.cat([s * torch.nn.functional.linear(x, A) for A, _, s in adapters], dim=1)
    assert_close_rel(t[:, : t_ref.shape[1]], t_ref, REL_BF16, "lora_shrink")
    y = ops.lora_linear_pre(xd, w.to(d, BF), None if b is None else b.to(d, BF), t, pk.b_cat,
                            None if res is None else res.to(d, BF))
    torch.cuda.synchronize()
    assert_close_rel(y, O.lora_linear(x, w, b, adapters, res), REL_BF16, "lora_linear_pre")
    # a column slice of a wider shrink result (layers sharing one input)
    wide = torch.zeros(M, pk.R + 64, dtype=BF, device=d)
    wide[:, 32:32 + pk.R] = t
    y2 = ops.lora_linear_pre(xd, w.to(d, BF), None if b is None else b.to(d, BF), wide[:, 32:32 + pk.R], pk.b_cat,
                             None if res is None else res.to(d, BF))
    assert torch.equal(y, y2)


def test_output_of_four_gib_takes_the_plain_store_path():
    """The GEMM epilogues store through a buffer descriptor with 32-bit offsets; an output of 4 GiB or more cannot be
    addressed that way and takes plain stores with 64-bit addresses.  M = 2^21 + 200 rows of 1024 columns (4.0 GiB):
    rows at the start, across the 4 GiB boundary and at the ragged end against the oracle, and the smaller problem made
    of the same rows bit for bit."""
    from katz_amd import ops

    say("4 GiB output")
    d = dev()
    M, N, K = (1 << 21) + 200, 1024, 64
    g = torch.Generator(device=d).manual_seed(12)
    x = (torch.randn(M, K, device=d, generator=g)).to(BF)
    w = (torch.randn(N, K, device=d, generator=g) * 0.1).to(BF)
    b = torch.randn(N, device=d, generator=g).to(BF)
    y = ops.lora_linear(x, w, b)
    assert y.numel() * 2 >= 1 << 32
    torch.cuda.synchronize()
    for r0 in (0, (1 << 21) - 300, M - 333):
        rows = slice(r0, r0 + 333)
        ref = O.lora_linear(x[rows].float().cpu(), w.float().cpu(), b.float().cpu(), [])
        assert_close_rel(y[rows], ref, REL_BF16, f"4 GiB output rows {r0}")
        assert torch.equal(y[rows][:128], ops.lora_linear(x[rows][:128].contiguous(), w, b))
    del y, x


def test_lora_linear_bf16_scale_zero_is_base():
    say("lora_linear_bf16 scale 0")
    x, w, b, adapters, _ = _lora_case(512, 640, 640, (64,), (0.0,), True, False, seed=3)
    y0 = _run_lora(x, w, b, adapters, None)
    y1 = _run_lora(x, w, b, [], None)
    assert torch.equal(y0, y1)


def test_kernels_are_bit_reproducible():
    """Same inputs, same bits, call after call: GEMM with LoRA + residual, GEGLU epilogue, attention."""
    from katz_amd import ops
    from katz_amd.layers import LoRALinear

    say("reproducibility")
    d = dev()
    g = torch.Generator().manual_seed(31)
    x = randn(g, 2048, 640).to(d, BF)
    lin = LoRALinear(640, 640).to(d, BF)
    lin.add_adapter("a", randn(g, 16, 640, std=0.05), randn(g, 640, 16, std=0.05))
    base = lin(x).clone()
    lin.set_active(["a"], [0.0])
    assert torch.equal(lin(x), base)           # scale 0 == no adapter, bit for bit
    lin.set_active(["a"], [1.0])
    y = lin(x, residual=base).clone()
    assert not torch.equal(lin(x), base)
    for _ in range(3):
        assert torch.equal(lin(x, residual=base), y)
    geg = LoRALinear(640, 5120, geglu=True).to(d, BF)
    geg.add_adapter("a", randn(g, 16, 640, std=0.05), randn(g, 5120, 16, std=0.05))
    geg.set_active(["a"], [0.7])
    y = geg(x).clone()
    assert torch.equal(geg(x), y)
    q = randn(g, 2, 1024, 640).to(d, BF)
    o = ops.attention(q, q, q, 10).clone()
    assert torch.equal(ops.attention(q, q, q, 10), o)


def test_lora_linear_bf16_geglu_epilogue():
    say("lora_linear_bf16 geglu")
    M, K, D = 2048, 1280, 5120
    x, w, b, adapters, _ = _lora_case(M, 2 * D, K, (64,), (1.0,), True, False, seed=5)
    y = _run_lora(x, w, b, adapters, None, geglu=True)
    proj = bf16_round(O.lora_linear(x, w, b, adapters))
    ref = O.geglu(proj)
    assert y.shape == (M, D)
    assert_close_rel(y, ref, REL_BF16, "geglu epilogue")


def test_lora_linear_f32_config1():
    """BASELINE config 1: x [2,4096,640], W [640,640], rank 32, scale 0.8, fp32, <= 1e-4."""
    from katz_amd import ops

    say("lora_linear_f32 config1")
    g = torch.Generator().manual_seed(0)
    x = torch.randn(2, 4096, 640, generator=g)
    w = torch.randn(640, 640, generator=g) * 0.02
    b = torch.randn(640, generator=g) * 0.02
    A = torch.randn(32, 640, generator=g) * 0.02
    Bm = torch.randn(640, 32, generator=g) * 0.02
    d = dev()
    cs = torch.full((32,), 0.8, dtype=torch.float32, device=d)
    y = ops.lora_linear(x.to(d), w.to(d), b.to(d), A.to(d), Bm.to(d).contiguous(), cs)
    torch.cuda.synchronize()
    ref = O.lora_linear(x.double(), w.double(), b.double(), [(A.double(), Bm.double(), 0.8)]).float()
    err = (y.cpu() - ref).abs().max().item()
    rel = err / ref.abs().max().item()
    assert y.shape == (2, 4096, 640)
    assert err <= 1e-4 and rel <= 1e-4, (err, rel)


def test_lora_linear_f32_ragged():
    from katz_amd import ops

    say("lora_linear_f32 ragged")
    g = torch.Generator().manual_seed(1)
    M, N, K, r = 70, 50, 37, 5
    x = torch.randn(M, K, generator=g); w = torch.randn(N, K, generator=g) * 0.1
    A = torch.randn(r, K, generator=g) * 0.1; Bm = torch.randn(N, r, generator=g) * 0.1
    res = torch.randn(M, N, generator=g)
    d = dev()
    cs = torch.full((r,), 1.5, dtype=torch.float32, device=d)
    y = ops.lora_linear(x.to(d), w.to(d), None, A.to(d), Bm.to(d), cs, residual=res.to(d))
    torch.cuda.synchronize()
    ref = O.lora_linear(x.double(), w.double(), None, [(A.double(), Bm.double(), 1.5)], res.double()).float()
    assert (y.cpu() - ref).abs().max().item() <= 1e-4


# ------------------------------------------------------------------------------------------- K3
ATTN_SHAPES = [
    # B, H, T, S
    (1, 2, 4096, 4096),   # self-attention at 64x64 (two of the ten heads)
    (2, 20, 1024, 1024),  # self-attention at 32x32, full head count
    (3, 16, 1000, 384),   # ragged last query block, six full key tiles
    (2, 10, 4096, 77),    # cross-attention at 64x64
    (2, 20, 1024, 77),    # cross-attention at 32x32
    (1, 1, 100, 77),      # ragged query block and key tile
    (2, 3, 130, 200),
    (1, 1, 1, 1),
]


@pytest.mark.parametrize("shape", ATTN_SHAPES, ids=lambda s: "B%dH%dT%dS%d" % s)
def test_attention_bf16(shape):
    from katz_amd import ops

    B, H, T, S = shape
    say("attention_bf16", shape)
    g = torch.Generator().manual_seed(7)
    q = randn(g, B, T, H * 64); k = randn(g, B, S, H * 64); v = randn(g, B, S, H * 64)
    d = dev()
    o = ops.attention(q.to(d, BF), k.to(d, BF), v.to(d, BF), H)
    torch.cuda.synchronize()
    ref = O.attention(q, k, v, H)
    assert_close_rel(o, ref, REL_BF16, "attention_bf16")


def test_attention_bf16_strided_views():
    """q/k/v as column slices of one fused [B,T,3*H*64] projection buffer."""
    from katz_amd import ops

    say("attention_bf16 strided")
    B, H, T = 2, 5, 333
    g = torch.Generator().manual_seed(8)
    qkv = randn(g, B, T, 3 * H * 64)
    d = dev()
    qkv_d = qkv.to(d, BF)
    q, k, v = qkv_d.split(H * 64, dim=-1)
    o = ops.attention(q, k, v, H)
    torch.cuda.synchronize()
    qr, kr, vr = qkv.split(H * 64, dim=-1)
    ref = O.attention(qr.contiguous(), kr.contiguous(), vr.contiguous(), H)
    assert_close_rel(o, ref, REL_BF16, "attention strided")


# ------------------------------------------------------------------------------------------- K4
GN_SHAPES = [
    # N, C, H, W, G
    (2, 320, 128, 128, 32),
    (2, 960, 64, 64, 32),
    (2, 1920, 32, 32, 32),
    (2, 2560, 32, 32, 32),
    (1, 32, 8, 8, 32),    # one channel per group
    (3, 64, 5, 8, 4),
]


@pytest.mark.parametrize("channels_last", [True, False], ids=["nhwc", "nchw"])
@pytest.mark.parametrize("act", ["silu", "none"])
@pytest.mark.parametrize("shape", GN_SHAPES, ids=lambda s: "N%dC%dH%dW%dG%d" % s)
def test_group_norm_bf16(shape, act, channels_last):
    from katz_amd import ops

    N, C, H, W, G = shape
    say("group_norm_bf16", shape, act, "nhwc" if channels_last else "nchw")
    g = torch.Generator().manual_seed(11)
    x = bf16_round(torch.randn(N, C, H, W, generator=g) * 2.0 + 3.0)  # non-zero mean: exercises the variance
    gamma = randn(g, C) + 1.0
    beta = randn(g, C, std=0.5)
    d = dev()
    xd = x.to(d, BF)
    if channels_last:
        xd = xd.contiguous(memory_format=torch.channels_last)
    eps = 1e-5 if act == "silu" else 1e-6
    y = ops.group_norm(xd, G, gamma.to(d, BF), beta.to(d, BF), eps, act)
    torch.cuda.synchronize()
    assert y.stride() == xd.stride()
    ref = O.group_norm(x, G, gamma, beta, eps, act)
    assert_close_rel(y, ref, REL_BF16, "group_norm_bf16")


def test_group_norm_no_affine():
    from katz_amd import ops

    say("group_norm no affine")
    g = torch.Generator().manual_seed(12)
    x = randn(g, 2, 64, 16, 16)
    d = dev()
    y = ops.group_norm(x.to(d, BF).contiguous(memory_format=torch.channels_last), 8, None, None, 1e-5, "none")
    torch.cuda.synchronize()
    assert_close_rel(y, O.group_norm(x, 8, None, None, 1e-5), REL_BF16, "group_norm no affine")


def test_group_norm_fused_channel_add():
    """norm(x + t[:, :, None, None]): the resnet's time-embedding add folded into the norm."""
    from katz_amd import ops

    say("group_norm add_nc")
    g = torch.Generator().manual_seed(14)
    d = dev()
    for (N, C, H, W, G), cl in [((2, 320, 32, 32, 32), True), ((2, 320, 32, 32, 32), False), ((2, 2560, 16, 16, 32), True)]:
        x = randn(g, N, C, H, W, std=2.0)
        t = randn(g, N, C)
        gamma = randn(g, C) + 1.0; beta = randn(g, C, std=0.5)
        xd = x.to(d, BF)
        if cl:
            xd = xd.contiguous(memory_format=torch.channels_last)
        y = ops.group_norm(xd, G, gamma.to(d, BF), beta.to(d, BF), 1e-5, "silu", add_nc=t.to(d, BF))
        torch.cuda.synchronize()
        ref = O.group_norm(x + t[:, :, None, None], G, gamma, beta, 1e-5, "silu")
        assert_close_rel(y, ref, REL_BF16, "group_norm add_nc")


def test_group_norm_is_deterministic():
    from katz_amd import ops

    x = torch.randn(2, 640, 64, 64, generator=torch.Generator().manual_seed(15)).to(dev(), BF)
    x = x.contiguous(memory_format=torch.channels_last)
    w = torch.ones(640, device=dev(), dtype=BF); b = torch.zeros(640, device=dev(), dtype=BF)
    y0 = ops.group_norm(x, 32, w, b, 1e-5, "silu").clone()
    for _ in range(3):
        assert torch.equal(ops.group_norm(x, 32, w, b, 1e-5, "silu"), y0)


def test_group_norm_unknown_activation_raises():
    from katz_amd import ops

    x = torch.zeros(1, 32, 8, 8, dtype=BF, device=dev())
    with pytest.raises(ValueError):
        ops.group_norm(x, 32, None, None, 1e-5, "relu")


@pytest.mark.parametrize("shape", [(8192, 640), (2048, 1280), (154, 2048), (5, 8), (3, 72)], ids=str)
def test_layer_norm_bf16(shape):
    from katz_amd import ops

    say("layer_norm_bf16", shape)
    M, D = shape
    g = torch.Generator().manual_seed(13)
    x = bf16_round(torch.randn(M, D, generator=g) * 1.5 + 0.7)
    gamma = randn(g, D) + 1.0
    beta = randn(g, D, std=0.3)
    d = dev()
    y = ops.layer_norm(x.to(d, BF), gamma.to(d, BF), beta.to(d, BF), 1e-5)
    torch.cuda.synchronize()
    assert_close_rel(y, O.layer_norm(x, gamma, beta, 1e-5), REL_BF16, "layer_norm_bf16")


# ------------------------------------------------------------------------------------------- K5
@pytest.mark.parametrize("approx", ["none", "tanh"])
@pytest.mark.parametrize("shape", [(2048, 5120), (8192, 2560), (7, 8)], ids=str)
def test_geglu_bf16(shape, approx):
    from katz_amd import ops

    say("geglu_bf16", shape, approx)
    M, D = shape
    g = torch.Generator().manual_seed(17)
    proj = randn(g, M, 2 * D, std=2.0)
    y = ops.geglu(proj.to(dev(), BF), approx)
    torch.cuda.synchronize()
    assert_close_rel(y, O.geglu(proj, approx), REL_BF16, "geglu_bf16")


def test_gelu_mul_bf16_matches_reference_argument_order():
    from katz_amd import ops

    say("gelu_mul_bf16")
    g = torch.Generator().manual_seed(18)
    x = randn(g, 3, 77, 40, std=2.0); m = randn(g, 3, 77, 40)
    y = ops.gelu_mul(x.to(dev(), BF), m.to(dev(), BF))
    torch.cuda.synchronize()
    assert_close_rel(y, O.gelu_mul(x, m, "tanh"), REL_BF16, "gelu_mul")


# ------------------------------------------------------------------------------------------- residuals
@pytest.mark.parametrize("k", [1, 3])
def test_residual_add_bf16(k):
    from katz_amd import ops

    say("residual_add_bf16", k)
    g = torch.Generator().manual_seed(19)
    d = dev()
    skip = randn(g, 2, 640, 64, 64)
    rs = [randn(g, 2, 640, 64, 64, std=0.1) for _ in range(k)]
    dst = skip.to(d, BF).contiguous(memory_format=torch.channels_last)
    rd = [r.to(d, BF).contiguous(memory_format=torch.channels_last) for r in rs]
    ops.residual_add_(dst, rd)
    torch.cuda.synchronize()
    ref = O.residual_add(skip, rs)
    if k == 1:
        # one ControlNet: a single rounding, identical to the bf16 add of the reference
        assert torch.equal(dst.cpu(), (skip.to(BF) + rs[0].to(BF)))
    assert_close_rel(dst, ref, REL_BF16, "residual_add")


@pytest.mark.parametrize("k", [0, 1, 2])
def test_concat_residual_bf16(k):
    from katz_amd import ops

    say("concat_residual_bf16", k)
    g = torch.Generator().manual_seed(23)
    d = dev()
    h = randn(g, 2, 1280, 32, 32); skip = randn(g, 2, 640, 32, 32)
    rs = [randn(g, 2, 640, 32, 32, std=0.1) for _ in range(k)]
    cl = lambda t: t.to(d, BF).contiguous(memory_format=torch.channels_last)
    out = ops.concat_residual(cl(h), cl(skip), [cl(r) for r in rs])
    torch.cuda.synchronize()
    assert out.shape == (2, 1920, 32, 32) and out.is_contiguous(memory_format=torch.channels_last)
    ref = O.concat_residual(h, skip, rs)
    if k <= 1:
        exp = torch.cat([h.to(BF), skip.to(BF) + rs[0].to(BF) if k else skip.to(BF)], dim=1)
        assert torch.equal(out.cpu(), exp)
    assert_close_rel(out, ref, REL_BF16, "concat_residual")


@pytest.mark.parametrize("shape", [(2, 1280, 32, 32), (2, 640, 64, 64), (1, 8, 1, 1), (3, 24, 5, 7)], ids=str)
def test_upsample_nearest2x(shape):
    """Upsample2D's interpolation (upsampling.py:169-171) is a copy: bit equality with F.interpolate on the same bf16
    values (the oracle's upsampler calls the same function)."""
    from katz_amd import ops

    say("upsample_nearest2x", shape)
    g = torch.Generator().manual_seed(sum(shape))
    x = randn(g, *shape).to(BF)
    out = ops.upsample_nearest2x(x.to(dev()).contiguous(memory_format=torch.channels_last))
    torch.cuda.synchronize()
    N, C, H, W = shape
    assert out.shape == (N, C, 2 * H, 2 * W) and out.is_contiguous(memory_format=torch.channels_last)
    assert torch.equal(out.cpu(), torch.nn.functional.interpolate(x, scale_factor=2.0, mode="nearest"))


# ------------------------------------------------------------------------------------------- K2
@pytest.mark.parametrize("T,K,N", [(1024, 1280, 1280), (4096, 640, 640), (77, 640, 640),
                                   (77, 2048, 640), (77, 2048, 1280),        # cross-attention to_k / to_v (context 2048)
                                   (1024, 1280, 10240), (1024, 5120, 1280)], ids=str)   # feed-forward in / out
def test_sgmv_heterogeneous_batch(T, K, N):
    """BASELINE config 4: 8 requests, each with its own adapter, ranks drawn (seed 2) from {8,16,32,64,128}, on every
    shape class of the SDXL attention linears (self-attention and to_out d x d, cross-attention to_k / to_v 2048 -> d)
    plus the feed-forward widths."""
    from katz_amd import ops

    say("sgmv", T, K, N)
    g = torch.Generator().manual_seed(2)
    n_req = 8
    choices = [8, 16, 32, 64, 128]
    ranks = [choices[i] for i in torch.randint(0, 5, (n_req,), generator=g).tolist()]
    seg_adapter = torch.randperm(n_req, generator=g).tolist()
    seg_adapter[3] = -1  # one request without an adapter
    x = randn(g, n_req * T, K)
    w = randn(g, N, K, std=0.02)
    adapters = [(randn(g, r, K, std=0.02), randn(g, N, r, std=0.02), 0.5 + 0.1 * i) for i, r in enumerate(ranks)]
    seg_start = [i * T for i in range(n_req + 1)]
    d = dev()
    RP = 128
    a_all = torch.zeros(n_req, RP, K); b_all = torch.zeros(n_req, N, RP)
    for i, (A, B, _) in enumerate(adapters):
        a_all[i, : A.shape[0]] = A
        b_all[i, :, : B.shape[1]] = B
    rank_pad = torch.tensor([(r + 31) // 32 * 32 for r in ranks], dtype=torch.int32, device=d)
    scales = torch.tensor([a[2] for a in adapters], dtype=torch.float32, device=d)
    ss = torch.tensor(seg_start, dtype=torch.int32, device=d)
    sa = torch.tensor(seg_adapter, dtype=torch.int32, device=d)
    xd = x.to(d, BF)
    y = ops.lora_linear(xd, w.to(d, BF))          # base projection, adapter-free
    y_base = y.clone()
    t = ops.sgmv_shrink(xd, a_all.to(d, BF), ss, sa, rank_pad, T)
    ops.sgmv_expand_(y, t, b_all.to(d, BF), ss, sa, rank_pad, scales, T)
    torch.cuda.synchronize()
    ref = O.sgmv(x, seg_start, seg_adapter, adapters, torch.nn.functional.linear(x, w))
    assert_close_rel(y, ref, REL_BF16, "sgmv")
    # the request without an adapter keeps the base projection bit for bit
    assert torch.equal(y[3 * T:4 * T], y_base[3 * T:4 * T])
    # shrink alone: t[:, :r] = x A^T
    a0 = seg_adapter[0]
    t_ref = torch.nn.functional.linear(x[:T], adapters[a0][0])
    assert_close_rel(t[:T, : ranks[a0]], t_ref, REL_BF16, "sgmv shrink")
    # both in one launch (t stays in the workgroup): same oracle, the adapter-free request untouched, and the two-launch
    # result to within the last bf16 place (the K order of the two products is the same; tiles differ)
    y2 = y_base.clone()
    ops.sgmv_fused_(y2, xd, a_all.to(d, BF), b_all.to(d, BF), ss, sa, rank_pad, scales, T)
    torch.cuda.synchronize()
    assert_close_rel(y2, ref, REL_BF16, "sgmv fused")
    assert torch.equal(y2[3 * T:4 * T], y_base[3 * T:4 * T])
    assert_close_rel(y2, y.float().cpu(), 1e-2, "sgmv fused vs two launches")


def test_sgmv_fused_ragged_segments_and_small_rank_pad():
    """Segments of unequal length (one empty, one shorter than a tile, one not a multiple of 128) and RP = 64."""
    from katz_amd import ops

    say("sgmv fused ragged")
    g = torch.Generator().manual_seed(11)
    lens = [300, 0, 77, 128, 513]
    K, N, RP = 640, 1280, 64
    ranks = [8, 64, 32, 16, 64]
    seg_adapter = [2, 0, -1, 4, 1]
    seg_start = [0]
    for n in lens:
        seg_start.append(seg_start[-1] + n)
    rows = seg_start[-1]
    x = randn(g, rows, K)
    base = randn(g, rows, N)
    adapters = [(randn(g, r, K, std=0.02), randn(g, N, r, std=0.02), 0.3 + 0.2 * i) for i, r in enumerate(ranks)]
    a_all = torch.zeros(len(ranks), RP, K); b_all = torch.zeros(len(ranks), N, RP)
    for i, (A, B, _) in enumerate(adapters):
        a_all[i, : A.shape[0]] = A
        b_all[i, :, : B.shape[1]] = B
    d = dev()
    rank_pad = torch.tensor([(r + 31) // 32 * 32 for r in ranks], dtype=torch.int32, device=d)
    scales = torch.tensor([a[2] for a in adapters], dtype=torch.float32, device=d)
    ss = torch.tensor(seg_start, dtype=torch.int32, device=d)
    sa = torch.tensor(seg_adapter, dtype=torch.int32, device=d)
    y = base.to(d, BF).clone()
    guard = y.clone()
    ops.sgmv_fused_(y, x.to(d, BF), a_all.to(d, BF), b_all.to(d, BF), ss, sa, rank_pad, scales, max(lens))
    torch.cuda.synchronize()
    ref = O.sgmv(x.to(BF).float(), seg_start, seg_adapter, adapters, base.to(BF).float())
    assert_close_rel(y, ref, REL_BF16, "sgmv fused ragged")
    assert torch.equal(y[seg_start[2]:seg_start[3]], guard[seg_start[2]:seg_start[3]])   # the request without an adapter


def test_sgmv_fused_grouped_layers_share_the_context():
    """kh_sgmv_fused_grouped_bf16: the to_k / to_v projections of several cross-attentions read the same 77-token text
    context per request (8 requests, each with its own adapter; one without), every layer with its own A / B / y, all in
    ONE launch: against the oracle per layer, and bit for bit against one kh_sgmv_fused_bf16 launch per layer."""
    from katz_amd import ops

    say("sgmv fused grouped")
    g = torch.Generator().manual_seed(23)
    n_req, T, K, N, RP, L = 8, 77, 2048, 1280, 128, 5
    ranks = [8, 128, 32, 64, 16, 128, 64, 32]
    seg_adapter = [3, 1, -1, 0, 7, 5, 2, 6]
    seg_start = [i * T for i in range(n_req + 1)]
    x = randn(g, n_req * T, K)
    d = dev()
    rank_pad = torch.tensor([(r + 31) // 32 * 32 for r in ranks], dtype=torch.int32, device=d)
    ss = torch.tensor(seg_start, dtype=torch.int32, device=d)
    sa = torch.tensor(seg_adapter, dtype=torch.int32, device=d)
    xd = x.to(d, BF)
    layers = []
    for l in range(L):
        adapters = [(randn(g, r, K, std=0.02), randn(g, N, r, std=0.02), 0.4 + 0.1 * i) for i, r in enumerate(ranks)]
        a_all = torch.zeros(n_req, RP, K); b_all = torch.zeros(n_req, N, RP)
        for i, (A, B, _) in enumerate(adapters):
            a_all[i, : A.shape[0]] = A
            b_all[i, :, : B.shape[1]] = B
        base = randn(g, n_req * T, N)
        layers.append((adapters, a_all.to(d, BF), b_all.to(d, BF), base))
    scales = torch.tensor([0.4 + 0.1 * i for i in range(n_req)], dtype=torch.float32, device=d)
    ys = [base.to(d, BF).clone() for (_, _, _, base) in layers]
    singles = [y.clone() for y in ys]
    table = ops.sgmv_fused_grouped_table(ys, [l[1] for l in layers], [l[2] for l in layers])
    ops.profile_begin()
    ops.sgmv_fused_grouped_(ys, xd, [l[1] for l in layers], [l[2] for l in layers], ss, sa, rank_pad, scales, T, table=table)
    launches = ops.profile_end()
    assert len(launches) == 1, launches                      # one launch for all layers
    for y1, (_, a_all, b_all, _) in zip(singles, layers):
        ops.sgmv_fused_(y1, xd, a_all, b_all, ss, sa, rank_pad, scales, T)
    torch.cuda.synchronize()
    for l, (adapters, _, _, base) in enumerate(layers):
        ref = O.sgmv(x.to(BF).float(), seg_start, seg_adapter, adapters, base.to(BF).float())
        assert_close_rel(ys[l], ref, REL_BF16, f"sgmv fused grouped, layer {l}")
        assert torch.equal(ys[l], singles[l]), f"layer {l}: grouped and single launches differ"
        assert torch.equal(ys[l][2 * T:3 * T], base.to(d, BF)[2 * T:3 * T])    # the request without an adapter


def test_sgmv_fused_many_column_tiles():
    """N = 5120 (40 column tiles): a workgroup takes at most five, whatever the row count; 4 requests x 200 rows."""
    from katz_amd import ops

    say("sgmv fused wide N")
    g = torch.Generator().manual_seed(29)
    n_req, T, K, N, RP = 4, 200, 640, 5120, 64
    ranks = [64, 16, 32, 8]
    seg_adapter = [1, 3, 0, 2]
    seg_start = [i * T for i in range(n_req + 1)]
    x, base = randn(g, n_req * T, K), randn(g, n_req * T, N)
    adapters = [(randn(g, r, K, std=0.02), randn(g, N, r, std=0.02), 0.5 + 0.1 * i) for i, r in enumerate(ranks)]
    a_all = torch.zeros(n_req, RP, K); b_all = torch.zeros(n_req, N, RP)
    for i, (A, B, _) in enumerate(adapters):
        a_all[i, : A.shape[0]] = A
        b_all[i, :, : B.shape[1]] = B
    d = dev()
    rank_pad = torch.tensor([(r + 31) // 32 * 32 for r in ranks], dtype=torch.int32, device=d)
    scales = torch.tensor([a[2] for a in adapters], dtype=torch.float32, device=d)
    y = base.to(d, BF).clone()
    ops.sgmv_fused_(y, x.to(d, BF), a_all.to(d, BF), b_all.to(d, BF), torch.tensor(seg_start, dtype=torch.int32, device=d),
                    torch.tensor(seg_adapter, dtype=torch.int32, device=d), rank_pad, scales, T)
    torch.cuda.synchronize()
    ref = O.sgmv(x.to(BF).float(), seg_start, seg_adapter, adapters, base.to(BF).float())
    assert_close_rel(y, ref, REL_BF16, "sgmv fused wide N")


def test_fused_qkv_matches_separate_projections():
    """Stacked to_q/to_k/to_v (n_split) with a shared shrink == three separate LoRA linears."""
    from katz_amd import ops
    from katz_amd.lora import Adapter, pack_adapters

    say("fused qkv")
    d = dev()
    g = torch.Generator().manual_seed(41)
    M, N, K = 1024, 640, 640
    x = randn(g, M, K)
    ws = [randn(g, N, K, std=0.02) for _ in range(3)]
    ads = [[(randn(g, 64, K, std=0.02), randn(g, N, 64, std=0.02), 0.8), (randn(g, 32, K, std=0.02), randn(g, N, 32, std=0.02), 0.6)]
           for _ in range(3)]
    packs = [pack_adapters({f"a{i}": Adapter(A, B, None, s) for i, (A, B, s) in enumerate(ad)}, ["a0", "a1"], K, N, BF, d)
             for ad in ads]
    R = packs[0].R
    xd = x.to(d, BF)
    t = ops.lora_shrink(xd, torch.cat([p.a_cat for p in packs]).contiguous(), torch.cat([p.col_scale for p in packs]).contiguous())
    y = ops.lora_linear_pre(xd, torch.cat([w.to(d, BF) for w in ws]).contiguous(), None, t,
                            torch.cat([p.b_cat for p in packs]).contiguous(), n_split=N)
    torch.cuda.synchronize()
    assert y.shape == (M, 3 * N) and t.shape == (M, 3 * R)
    for j in range(3):
        ref = O.lora_linear(x, ws[j], None, ads[j])
        assert_close_rel(y[:, j * N:(j + 1) * N], ref, REL_BF16, f"fused qkv part {j}")


@pytest.mark.parametrize("shape", [
    # (Nb, Cin, H, W, Cout, stride, bias, residual)
    (2, 64, 16, 16, 64, 1, True, False),
    (2, 320, 32, 32, 320, 1, True, True),      # 128-row tiles cross image rows
    (1, 96, 13, 9, 40, 1, True, False),        # ragged: M and Cout not multiples of the tile, Cin = 3 x 32
    (2, 128, 16, 16, 128, 2, True, False),     # Downsample2D
    (1, 64, 15, 11, 72, 2, False, True),       # odd sizes, stride 2
    (2, 1280, 32, 32, 1280, 1, True, True),    # the deepest SDXL resnet conv (64x160 tiles, waves split K)
    (2, 640, 64, 64, 640, 1, True, True),      # the middle level (128x160 tiles, waves split K)
    (1, 640, 60, 67, 640, 1, True, False),     # same tiles, ragged M (4020 pixels), rows crossing image rows
    (2, 1280, 31, 31, 1280, 1, False, True),   # 64x160 tiles, ragged M (1922 pixels)
    (2, 640, 50, 80, 640, 1, True, True),      # 128x160 tiles, ragged M (8000 pixels)
])
def test_conv3x3_nhwc_bf16(shape):
    """Implicit-GEMM 3x3 convolution against torch's fp32 conv2d on the same bf16-rounded operands."""
    from katz_amd import ops

    Nb, Cin, H, W, Cout, stride, has_bias, has_res = shape
    say("conv3x3", shape)
    d = dev()
    g = torch.Generator().manual_seed(7 + Cin + Cout)
    x = randn(g, Nb, Cin, H, W).to(BF)
    w = randn(g, Cout, Cin, 3, 3, std=(9 * Cin) ** -0.5).to(BF)
    b = randn(g, Cout).to(BF) if has_bias else None
    ref = torch.nn.functional.conv2d(x.float(), w.float(), None if b is None else b.float(), stride=stride, padding=1)
    res = randn(g, *ref.shape).to(BF) if has_res else None
    if res is not None:
        ref = ref.to(BF).float() + res.float()   # the kernel rounds the conv to bf16 before the residual add
    xd = x.to(d).contiguous(memory_format=torch.channels_last)
    y = ops.conv3x3(xd, ops.pack_conv3x3_weight(w.to(d)), None if b is None else b.to(d), stride=stride,
                    residual=None if res is None else res.to(d).contiguous(memory_format=torch.channels_last))
    torch.cuda.synchronize()
    assert y.shape == ref.shape and y.is_contiguous(memory_format=torch.channels_last)
    assert_close_rel(y, ref, REL_BF16, f"conv3x3 {shape}")


@pytest.mark.parametrize("lat_f32", [False, True])
def test_cfg_euler_step_kernel(lat_f32):
    """Fused guidance + Euler step against (a) the same formula in fp32 on the bf16-rounded inputs (tight) and
    (b) the oracle's torch-semantics step on bf16 tensors (bf16 tolerance)."""
    from katz_amd import ops
    from oracle.euler import EulerDiscreteScheduler as OSched, classifier_free_guidance

    say("cfg_euler", lat_f32)
    d = dev()
    g = torch.Generator().manual_seed(3)
    sch = OSched(beta_start=0.00085, beta_end=0.012, beta_schedule="scaled_linear", timestep_spacing="leading", steps_offset=1)
    sch.set_timesteps(50)
    i = 7
    sigma, sigma_next = sch.sigmas[i], sch.sigmas[i + 1]
    noise = randn(g, 2, 4, 32, 32).to(BF)
    lat = (randn(g, 1, 4, 32, 32) * sigma).to(torch.float32 if lat_f32 else BF)
    gs = 7.5
    # (a) fp32 restatement
    u, t = noise[:1].float(), noise[1:].float()
    eps = u + gs * (t - u)
    x = lat.float()
    x0 = x - sigma * eps
    prev = x + ((x - x0) / sigma) * (sigma_next - sigma)
    den = (sigma_next ** 2 + 1) ** 0.5
    coef = torch.tensor([sigma.item(), sigma_next.item(), den.item()], dtype=torch.float32, device=d)
    nxt = torch.empty(2, 4, 32, 32, dtype=BF, device=d)
    out = ops.cfg_euler_step(noise.to(d), lat.to(d), coef, gs, model_input_next=nxt)
    torch.cuda.synchronize()
    assert out.dtype == lat.dtype
    ref = prev if lat_f32 else prev.to(BF)
    err = (out.float().cpu() - ref.float()).abs().max().item()
    # fp32 latents: rounding-order noise only; bf16 latents: at most one bf16 ulp where that noise crosses a tie
    assert err <= (1e-5 if lat_f32 else 2.0 ** -8) * max(1.0, prev.abs().max().item()), err
    if not lat_f32:
        assert (out.cpu() != ref).float().mean().item() < 1e-2
    ref_next = (ref.float() / den).to(BF)
    assert torch.equal(nxt[0].cpu(), ref_next[0]) or (nxt[0].float().cpu() - ref_next[0].float()).abs().max() <= 2 ** -7 * ref_next.abs().max()
    assert torch.equal(nxt[0], nxt[1])
    # (b) the reference's op sequence on bf16 tensors (rounds eps and sigma*eps to bf16 on the way)
    sch.step_index = i
    o2 = sch.step(classifier_free_guidance(noise, gs), sch.timesteps[i], lat.to(BF))
    assert_close_rel(out, o2.reshape(out.shape), REL_BF16, "cfg+euler vs oracle op sequence")


@pytest.mark.parametrize("lat_f32", [True, False])
def test_denoise_loop_matches_oracle_loop(lat_f32):
    """50 guided Euler steps around a cheap elementwise 'model' with bf16 input / output (what the UNet is to the
    loop): the product loop (fused kernel) against the oracle's loop.  With fp32 latents the two differ by
    rounding order only; with the reference's model-dtype (bf16) latents every step re-rounds the state, so 50
    steps of independent bf16 roundings bound the agreement (cosine, and 10 % of |ref| + rms elementwise)."""
    from katz_amd.scheduler import EulerDiscreteScheduler, denoise_loop
    from oracle.euler import EulerDiscreteScheduler as OSched, denoise_loop as oracle_loop

    say("denoise loop", lat_f32)
    d = dev()
    cfg = dict(beta_start=0.00085, beta_end=0.012, beta_schedule="scaled_linear", timestep_spacing="leading", steps_offset=1)
    ps, os_ = EulerDiscreteScheduler(**cfg), OSched(**cfg)
    ps.set_timesteps(50, device=d)
    os_.set_timesteps(50)
    assert torch.equal(ps.timesteps.cpu(), os_.timesteps) and torch.equal(ps.sigmas, os_.sigmas)
    assert ps.init_noise_sigma.item() == os_.init_noise_sigma.item()
    g = torch.Generator().manual_seed(5)
    lat0 = (randn(g, 1, 4, 16, 16) * os_.init_noise_sigma).to(BF)

    def model(x, t):  # rows: uncond, text; a smooth, contracting elementwise map of the bf16-rounded input
        x = x.to(BF).float()
        scale = torch.tensor([[[[0.8]]], [[[1.1]]]], dtype=torch.float32, device=x.device)
        y = x / (1.0 + x.abs()) * scale * (1.0 - t.float() / 2000.0)
        return y.to(BF)

    got = denoise_loop(model, ps, lat0.to(d), 7.5, latents_fp32=lat_f32)
    ref = oracle_loop(lambda x, t: model(x, t).to(x.dtype), os_, lat0.float() if lat_f32 else lat0, 7.5)
    torch.cuda.synchronize()
    assert got.dtype == (torch.float32 if lat_f32 else BF)
    cos = torch.nn.functional.cosine_similarity(got.float().cpu().flatten(), ref.float().flatten(), dim=0).item()
    assert cos >= 0.999, cos
    assert_close_rel(got, ref, 1e-2 if lat_f32 else 1e-1, "50-step loop")


@pytest.mark.parametrize("stride", [1, 2])
def test_conv3x3_with_lora_adapters(stride):
    """Conv3x3 with two active LoRA adapters against the oracle's LoRA conv; scale 0, disable and delete restore the base."""
    from katz_amd.layers import Conv3x3

    say("conv lora", stride)
    d = dev()
    g = torch.Generator().manual_seed(17)
    cin, cout = 64, 96
    conv = Conv3x3(cin, cout, stride=stride)
    with torch.no_grad():
        conv.weight.copy_(randn(g, cout, cin, 3, 3, std=(9 * cin) ** -0.5).to(BF).float())
        conv.bias.copy_(randn(g, cout).to(BF).float())
    w, b = conv.weight.detach().clone(), conv.bias.detach().clone()
    conv = conv.to(d, BF)
    ads = [(randn(g, 8, cin, 3, 3, std=0.05).to(BF).float(), randn(g, cout, 8, 1, 1, std=0.05).to(BF).float(), 16.0, 0.8),
           (randn(g, 4, cin, 3, 3, std=0.05).to(BF).float(), randn(g, cout, 4, 1, 1, std=0.05).to(BF).float(), None, 0.6)]
    for i, (A, B, alpha, wgt) in enumerate(ads):
        conv.add_adapter(f"a{i}", A, B, alpha)
    conv.set_active(["a0", "a1"], [0.8, 0.6])
    x = randn(g, 2, cin, 12, 10).to(BF)
    xd = x.to(d).contiguous(memory_format=torch.channels_last)
    with torch.no_grad():
        y = conv(xd)
        ref = O.lora_conv2d(x.float(), w, b, [(ads[0][0], ads[0][1], 0.8 * 16.0 / 8), (ads[1][0], ads[1][1], 0.6)], stride=stride)
        base = O.lora_conv2d(x.float(), w, b, [], stride=stride)
        torch.cuda.synchronize()
        assert y.shape == ref.shape
        assert_close_rel(y, ref, REL_BF16, "conv + lora")
        assert (ref - base).abs().max() > 0.05   # the adapters matter at this scale
        conv.set_active(["a0", "a1"], [0.0, 0.0])
        assert_close_rel(conv(xd), base, REL_BF16, "conv + lora at scale 0")
        conv.set_active(["a0", "a1"], [0.8, 0.6])
        conv.adapters_enabled = False
        conv.refresh_adapters()
        y_dis = conv(xd)
        conv.adapters_enabled = True
        conv.delete_adapter("a0"); conv.delete_adapter("a1")
        assert torch.equal(conv(xd), y_dis)
        assert_close_rel(y_dis, base, REL_BF16, "conv, adapters disabled")


def test_conv1x1_with_lora_and_conv_fuse():
    """The resnets' 1x1 conv_shortcut with two LoRA adapters (LoRAConv2dLayer, models/lora.py:258-296) against the
    oracle, and fuse / unfuse of 1x1 and 3x3 conv adapters (merged kernel, :403-441): fused == unfused == oracle."""
    from katz_amd.layers import Conv1x1, Conv3x3

    say("conv1x1 lora + conv fuse")
    d = dev()
    g = torch.Generator().manual_seed(23)
    cin, cout = 64, 128
    x = randn(g, 2, cin, 12, 10).to(BF)
    xd = x.to(d).contiguous(memory_format=torch.channels_last)
    for cls, k in ((Conv1x1, 1), (Conv3x3, 3)):
        conv = cls(cin, cout)
        with torch.no_grad():
            conv.weight.copy_(randn(g, cout, cin, k, k, std=(k * k * cin) ** -0.5).to(BF).float())
            conv.bias.copy_(randn(g, cout).to(BF).float())
        w, b = conv.weight.detach().clone(), conv.bias.detach().clone()
        conv = conv.to(d, BF)
        ads = [(randn(g, 8, cin, k, k, std=0.08).to(BF).float(), randn(g, cout, 8, 1, 1, std=0.08).to(BF).float(), 16.0, 0.8),
               (randn(g, 4, cin, k, k, std=0.08).to(BF).float(), randn(g, cout, 4, 1, 1, std=0.08).to(BF).float(), None, 0.6)]
        for i, (A, B, alpha, wgt) in enumerate(ads):
            conv.add_adapter(f"a{i}", A, B, alpha)
        conv.set_active(["a0", "a1"], [0.8, 0.6])
        oracle_ads = [(ads[0][0], ads[0][1], 0.8 * 16.0 / 8), (ads[1][0], ads[1][1], 0.6)]
        with torch.no_grad():
            ref = O.lora_conv2d(x.float(), w, b, oracle_ads, padding=k // 2)
            base = O.lora_conv2d(x.float(), w, b, [], padding=k // 2)
            y = conv(xd)
            assert_close_rel(y, ref, REL_BF16, f"conv{k}x{k} + lora")
            assert (ref - base).abs().max() > 0.05
            conv.fuse()
            assert set(conv._fused) == {"a0", "a1"}
            merged = w + sum(s * (B.reshape(cout, -1) @ A.reshape(A.shape[0], -1)).reshape(w.shape) for A, B, s in oracle_ads)
            assert_close_rel(conv.weight.float().cpu(), merged, 1e-2, "merged conv weight")
            yf = conv(xd)
            assert_close_rel(yf, ref, REL_BF16, f"conv{k}x{k} fused")
            conv.unfuse()
            assert_close_rel(conv.weight.float().cpu(), w, 1e-2, "unfused conv weight")
            assert_close_rel(conv(xd), ref, REL_BF16, f"conv{k}x{k} unfused again")
            conv.set_active([])
            assert_close_rel(conv(xd), base, REL_BF16, f"conv{k}x{k} without adapters")


@pytest.mark.parametrize("cin,cout", [(4, 64), (64, 4), (3, 16), (16, 32)])
def test_conv3x3_module_pads_small_channel_counts(cin, cout):
    """Conv3x3 on the katz_hip kernel for the UNet's conv_in / conv_out and the ControlNet's image embedding:
    channel counts below the kernel's granule are zero-padded, results match F.conv2d, and are bit-reproducible."""
    from katz_amd.layers import Conv3x3

    say("conv small channels", cin, cout)
    d = dev()
    g = torch.Generator().manual_seed(cin * 100 + cout)
    conv = Conv3x3(cin, cout)
    with torch.no_grad():
        conv.weight.copy_(randn(g, cout, cin, 3, 3, std=(9 * cin) ** -0.5).to(BF).float())
        conv.bias.copy_(randn(g, cout).to(BF).float())
    x = randn(g, 2, cin, 20, 12).to(BF)
    ref = torch.nn.functional.conv2d(x.float(), conv.weight.detach(), conv.bias.detach(), padding=1)
    conv = conv.to(d, BF)
    from katz_amd import ops
    ops.CALL_LOG = []
    try:
        with torch.no_grad():
            y = conv(x.to(d))
            y2 = conv(x.to(d))
    finally:
        log, ops.CALL_LOG = ops.CALL_LOG, None
    torch.cuda.synchronize()
    assert [c[0] for c in log] == ["conv3x3", "conv3x3"], "the module must run the katz_hip kernel"
    assert y.shape == ref.shape and torch.equal(y, y2)
    assert_close_rel(y, ref, REL_BF16, "conv3x3 with padded channels")


@pytest.mark.parametrize("tile", [0, 16, 20, 27, 28, 32, 40, 41])
@pytest.mark.parametrize("shape", [(384, 512, 256, 64), (1000, 328, 640, 0), (2048, 1280, 1280, 128),
                                   (6600, 640, 640, 128), (1000, 1280, 2560, 64), (70, 168, 64, 0)])
def test_pipelined_gemm_tile_variants(tile, shape):
    """Every tile configuration of the pipelined kernel and of the K-splitting 160-column kernel (codes 40, 41),
    plain and with the rank columns as extra K tiles, bias, residual, ragged M / N, against the oracle.  Code 0 is
    the automatic choice: the fourth and fifth shape are ones it sends to the 160-column kernel."""
    from katz_amd import ops

    M, N, K, R = shape
    say("tile variant", tile, shape)
    d = dev()
    g = torch.Generator().manual_seed(tile * 7 + M)
    x, w, b, res = randn(g, M, K), randn(g, N, K, std=0.03), randn(g, N), randn(g, M, N)
    xd, wd, bd, rd = (t.to(d, BF) for t in (x, w, b, res))
    if R == 0:
        y = ops.lora_linear(xd, wd, bd, residual=rd, tile=tile)
        ref = O.lora_linear(xd.float().cpu(), wd.float().cpu(), bd.float().cpu(), [], residual=rd.float().cpu())
    else:
        A, B = randn(g, R, K, std=0.05), randn(g, N, R, std=0.05)
        Ad, Bd = A.to(d, BF), B.to(d, BF)
        t = ops.lora_shrink(xd, Ad, torch.full((R,), 0.7, device=d))
        y = ops.lora_linear_pre(xd, wd, bd, t, Bd, residual=rd, tile=tile)
        ref = O.lora_linear(xd.float().cpu(), wd.float().cpu(), bd.float().cpu(), [(Ad.float().cpu(), Bd.float().cpu(), 0.7)],
                            residual=rd.float().cpu())
    torch.cuda.synchronize()
    assert_close_rel(y, ref, REL_BF16, f"tile {tile} {shape}")


@pytest.mark.parametrize("shape", [(256, 320, 64, 0), (512, 640, 192, 64), (2048, 10240, 1280, 128)])
@pytest.mark.parametrize("geglu", [False, True])
def test_wide_tile_gemm(shape, geglu):
    """The 256x320-tile kernel (code 42; the automatic choice for the third shape): plain and with the rank columns
    as extra K tiles, bias, residual or the GEGLU epilogue, against the oracle; and bit for bit against the 128x128
    pipelined kernel, whose summation order per output element it shares."""
    from katz_amd import ops
    from katz_amd.lora import interleave_geglu_rows

    M, N, K, R = shape
    say("wide tile", shape, geglu)
    d = dev()
    g = torch.Generator().manual_seed(M + N + int(geglu))
    x, w, b = randn(g, M, K), randn(g, N, K, std=0.03), randn(g, N)
    res = None if geglu else randn(g, M, N)
    xd = x.to(d, BF)
    wd = (interleave_geglu_rows(w) if geglu else w).to(d, BF)
    bd = (interleave_geglu_rows(b) if geglu else b).to(d, BF)
    rd = None if res is None else res.to(d, BF)
    ads = []
    if R == 0:
        run = lambda tile: ops.lora_linear(xd, wd, bd, residual=rd, geglu=geglu, tile=tile)
    else:
        A, B = randn(g, R, K, std=0.05), randn(g, N, R, std=0.05)
        Ad = A.to(d, BF)
        Bd = (interleave_geglu_rows(B) if geglu else B).to(d, BF)
        t = ops.lora_shrink(xd, Ad, torch.full((R,), 0.7, device=d))
        run = lambda tile: ops.lora_linear_pre(xd, wd, bd, t, Bd, residual=rd, geglu=geglu, tile=tile)
        ads = [(Ad.float().cpu(), B.to(BF).float(), 0.7)]
    y = run(42)
    y16 = run(16)
    y0 = run(0)
    torch.cuda.synchronize()
    assert torch.equal(y, y16), "wide tile differs from the 128x128 kernel"
    assert torch.equal(y0, y16), "automatic choice differs from the 128x128 kernel"
    xf, wf, bf = xd.float().cpu(), w.to(BF).float(), b.to(BF).float()
    if geglu:
        ref = O.geglu(bf16_round(O.lora_linear(xf, wf, bf, ads)))
    else:
        ref = O.lora_linear(xf, wf, bf, ads, residual=rd.float().cpu())
    assert_close_rel(y, ref, REL_BF16, f"wide tile {shape} geglu={geglu}")


def test_wide_tile_geglu_gate_range():
    """GEGLU epilogue of the 256x320-tile kernel on gates outside and at the edges of its lookup table (zero, tiny,
    2^-15, just below 32, huge, infinite): x = 0, so the projection is the bias."""
    from katz_amd import ops
    from katz_amd.lora import interleave_geglu_rows

    say("wide tile geglu gate range")
    d = dev()
    M, K, D = 256, 64, 320
    specials = torch.tensor([0.0, -0.0, 1e-6, -1e-6, 2.0 ** -15, -(2.0 ** -15), 2.0 ** -15 * 0.99, 31.875, -31.875, 32.0,
                             -32.0, 40.0, -40.0, 1e30, -1e30, float("inf"), -float("inf"), 0.5, -0.5, 3.0, -3.0])
    g = torch.Generator().manual_seed(3)
    gate = randn(g, D) * 2.0
    gate[: specials.numel()] = specials
    value = randn(g, D)
    b = torch.cat([value, gate]).to(BF)                       # reference layout: value rows, then gate rows
    w = torch.zeros(2 * D, K)
    x = torch.zeros(M, K)
    wd, bd = interleave_geglu_rows(w).to(d, BF), interleave_geglu_rows(b).to(d, BF)
    y = ops.lora_linear(x.to(d, BF), wd, bd, geglu=True, tile=42)
    y16 = ops.lora_linear(x.to(d, BF), wd, bd, geglu=True, tile=16)
    torch.cuda.synchronize()
    assert torch.equal(y.view(torch.int16), y16.view(torch.int16)), "lookup differs from the direct evaluation"
    ref = O.geglu(b.float().unsqueeze(0).expand(M, -1).contiguous())
    fin = torch.isfinite(ref[0])
    assert_close_rel(y[:, fin], ref[:, fin], REL_BF16, "wide tile geglu gate range")


@pytest.mark.parametrize("case", [
    # (M, N, K, residual, n_split)
    (2048, 1280, 1280, True, 0),       # the d x d layers: 160 GEMM + 32 shrink workgroups
    (2048, 1280, 5120, True, 0),       # ff.net.2
    (1990, 1280, 1280, False, 0),      # ragged rows: the last shrink tile is partly out of range
    (2048, 3840, 1280, False, 1280),   # stacked q / k / v: T = [M, 3 x 128], one 64 x 96 tile per layer and 64 rows
    # the GEMM's 128 x 160 tiles fill the chip: every workgroup computes a 32 x 96 piece of T before its tile
    (8192, 640, 640, True, 0),
    (8192, 640, 2560, True, 0),        # ff.net.2 at the 64 x 64 level
    (8100, 640, 640, False, 0),        # ragged rows: the last row block's fourth quarter is partly out of range
])
def test_lora_linear_split_rank_96_of_128(case):
    """Two adapters of ranks 64 + 32 packed into 128 rank columns of which the last 32 are padding (r_used = 96): the
    in-launch shrink then runs on 64 x 96 tiles and leaves T's padding columns unwritten, which the GEMM tiles never
    multiply (the cooperative form of the 8192-row cases zeroes them instead).  T is poisoned with NaNs first; results
    against the oracle, against the two-launch form and (bit for bit, where the call that does not know about the
    padding also shrinks inside its launch) against that call."""
    from katz_amd import ops

    M, N, K, has_res, n_split = case
    R, RU = 128, 96
    say("lora_linear_split r_used 96", case)
    d = dev()
    g = torch.Generator().manual_seed(M + N + K + 96)
    parts = N // n_split if n_split else 1
    x, w, b = randn(g, M, K), randn(g, N, K, std=0.03), randn(g, N)
    A, B = randn(g, parts * R, K, std=0.05), randn(g, N, R, std=0.05)
    for j in range(parts):
        A[j * R + RU:(j + 1) * R] = 0
    B[:, RU:] = 0
    res = randn(g, M, N) if has_res else None
    xd, wd, bd, Ad, Bd = (t.to(d, BF) for t in (x, w, b, A, B))
    rd = None if res is None else res.to(d, BF)
    cs = torch.full((parts * R,), 0.7, device=d)
    assert ops._lib.load().kh_lora_linear_split_launches(M, N, K, R, n_split, (RU // 16) << 16) == 1
    # every scratch buffer torch hands out next is full of NaNs: what the shrink does not write must never be read
    for _ in range(3):
        junk = torch.full((M, parts * R), float("nan"), device=d, dtype=BF)
        del junk
    ops.split_counters_reset(d)
    y = ops.lora_linear_split(xd, wd, bd, Ad, cs, Bd, residual=rd, n_split=n_split, r_used=RU)
    flag = ops.split_counters_last(d)[-1:].clone()
    y_again = ops.lora_linear_split(xd, wd, bd, Ad, cs, Bd, residual=rd, n_split=n_split, r_used=RU)
    y_two = ops.lora_linear_split(xd, wd, bd, Ad, cs, Bd, residual=rd, n_split=n_split, r_used=RU, two_launches=True)
    y_full = ops.lora_linear_split(xd, wd, bd, Ad, cs, Bd, residual=rd, n_split=n_split)
    torch.cuda.synchronize()
    assert int(flag) == 0 and torch.isfinite(y.float()).all()
    assert torch.equal(y, y_again)
    if ops._lib.load().kh_lora_linear_split_launches(M, N, K, R, n_split, 0) == 1:
        assert torch.equal(y, y_full)
    else:   # without the promise these shapes take two launches
        assert (y != y_full).float().mean().item() < 5e-3
    # the two-launch form differs only by the fp32 summation order inside the shrink: a handful of last-bit differences
    assert (y != y_two).float().mean().item() < 5e-3
    xf, wf, bfl, Af, Bf = (t.float().cpu() for t in (xd, wd, bd, Ad, Bd))
    step = n_split if n_split else N
    for j in range(parts):
        rows = slice(j * step, (j + 1) * step)
        ref = O.lora_linear(xf, wf[rows], bfl[rows], [(Af[j * R:(j + 1) * R], Bf[rows], 0.7)],
                            residual=None if rd is None else rd.float().cpu()[:, rows])
        assert_close_rel(y[:, rows], ref, REL_BF16, f"split r_used 96 {case} part {j}")
    ops.check_split_timeouts(d)


@pytest.mark.parametrize("M", [8192, 8100, 4096])
@pytest.mark.parametrize("fold", [False, True], ids=["plain", "ln-fold"])
def test_stacked_layers_rank_96_shrink_as_its_own_launch(M, fold):
    """q / k / v of the 64 x 64 level: three stacked layers, rank 96 of 128 each, on GEMM tiles that fill the chip in several
    rounds, so the shrink stays a launch of its own -- on 128-row x 96-column tiles, one per layer and 128 rows, that skip
    the padding columns and zero them in T.  T is poisoned with NaNs first.  Against the oracle and against the call
    without the promise (64 x 64 tiles over all 384 columns: another summation order)."""
    from katz_amd import ops
    from katz_amd.lora import fold_layer_norm

    N, K, n_split, R, RU = 1920, 640, 640, 128, 96
    say("stacked rank-96 shrink", M, fold)
    d = dev()
    g = torch.Generator().manual_seed(M + 17)
    x, w, b = randn(g, M, K), randn(g, N, K, std=0.03), randn(g, N, std=0.1)
    A, B = randn(g, 3 * R, K, std=0.05), randn(g, N, R, std=0.05)
    for j in range(3):
        A[j * R + RU:(j + 1) * R] = 0
    B[:, RU:] = 0
    cs = torch.full((3 * R,), 0.7, device=d)
    assert ops._lib.load().kh_lora_linear_split_launches(M, N, K, R, n_split, (RU // 16) << 16) == 2
    xd, wd, bd, Ad, Bd = (t.to(d, BF) for t in (x, w, b, A, B))
    if fold:
        gamma, beta = randn(g, K, std=0.2) + 1.0, randn(g, K, std=0.2)
        wp, c1, c2, ap, ca1, ca2 = fold_layer_norm(wd, bd, gamma.to(d, BF), beta.to(d, BF), Ad)
        st = torch.zeros((ops.LN_SLOTS, M, 2), dtype=torch.float32, device=d)
        st[0, :, 0] = xd.float().sum(-1)
        st[0, :, 1] = (xd.float() ** 2).sum(-1)
        run = lambda ru: ops.lora_linear_norm(xd, wp, None, ap, cs, Bd, n_split=n_split, r_used=ru, ln=(st, c1, c2, ca1, ca2, 1e-5))
        xn = O.layer_norm(xd.float().cpu(), gamma.to(BF).float(), beta.to(BF).float(), 1e-5)
    else:
        run = lambda ru: ops.lora_linear_split(xd, wd, bd, Ad, cs, Bd, n_split=n_split, r_used=ru)
        xn = xd.float().cpu()
    for _ in range(3):   # what torch hands out next is full of NaNs
        junk = torch.full((M, 3 * R), float("nan"), device=d, dtype=BF)
        del junk
    y = run(RU)
    y_again = run(RU)
    y_full = run(0)
    torch.cuda.synchronize()
    assert torch.isfinite(y.float()).all() and torch.equal(y, y_again)
    assert (y != y_full).float().mean().item() < 5e-3
    wf, bfl, Af, Bf = (t.float().cpu() for t in (wd, bd, Ad, Bd))
    for j in range(3):
        rows = slice(j * n_split, (j + 1) * n_split)
        ref = O.lora_linear(xn, wf[rows], bfl[rows], [(Af[j * R:(j + 1) * R], Bf[rows], 0.7)])
        assert_close_rel(y[:, rows], ref, REL_BF16, f"stacked rank-96 shrink part {j}")


@pytest.mark.parametrize("case", [
    # (M, N, K, R, residual, n_split)
    (2048, 1280, 1280, 128, True, 0),      # to_out / attn2.to_q at 32x32: 160 GEMM + 64 shrink workgroups in one launch
    (2048, 1280, 1280, 64, False, 0),
    (2000, 1280, 640, 64, True, 0),        # ragged rows: the last 128-row block has one 64-row shrink tile
    (1100, 1000, 1280, 128, True, 0),      # ragged rows and columns
    (2048, 1280, 5120, 128, True, 0),      # ff.net.2
    (2048, 3840, 1280, 128, False, 1280),  # stacked q / k / v: one launch on 256x128 tiles, T = [M, 3R]
    (1900, 3840, 1280, 64, False, 1280),   # the same, ragged rows (the last 256-row block has 2 of 4 shrink tiles)
    (8192, 640, 640, 128, True, 0),        # every CU busy with the GEMM: two launches
])
def test_lora_linear_split(case):
    """kh_lora_linear_split_bf16 (shrink inside the GEMM launch where the rule allows, else two launches): against the
    oracle, against the forced two-launch form, repeated calls bit for bit (each on fresh counters from the arena,
    also across an arena reset), the time-out flag clear."""
    from katz_amd import ops

    M, N, K, R, has_res, n_split = case
    say("lora_linear_split", case)
    d = dev()
    g = torch.Generator().manual_seed(M + N + K + R)
    parts = N // n_split if n_split else 1
    x, w, b = randn(g, M, K), randn(g, N, K, std=0.03), randn(g, N)
    A, B = randn(g, parts * R, K, std=0.05), randn(g, N, R, std=0.05)
    res = randn(g, M, N) if has_res else None
    xd, wd, bd, Ad, Bd = (t.to(d, BF) for t in (x, w, b, A, B))
    rd = None if res is None else res.to(d, BF)
    cs = torch.full((parts * R,), 0.7, device=d)
    run = lambda **kw: ops.lora_linear_split(xd, wd, bd, Ad, cs, Bd, residual=rd, n_split=n_split, **kw)
    ys, flags = [], []
    for i in range(4):
        if i == 2:
            ops.split_counters_reset(d)          # what the UNet forward does once per step
        ys.append(run())
        flags.append(ops.split_counters_last(d)[-1:].clone())
    y2 = run(two_launches=True)
    torch.cuda.synchronize()
    assert all(int(f) == 0 for f in flags), "a bounded wait inside a launch ran out"
    for y in ys[1:]:
        assert torch.equal(y, ys[0])
    xf, wf, bfl, Af, Bf = (t.float().cpu() for t in (xd, wd, bd, Ad, Bd))
    step = n_split if n_split else N
    for j in range(parts):   # every stacked layer against the oracle with its own A / B
        rows = slice(j * step, (j + 1) * step)
        ref = O.lora_linear(xf, wf[rows], bfl[rows], [(Af[j * R:(j + 1) * R], Bf[rows], 0.7)],
                            residual=None if rd is None else rd.float().cpu()[:, rows])
        assert_close_rel(ys[0][:, rows], ref, REL_BF16, f"split {case} part {j}")
        assert_close_rel(y2[:, rows], ref, REL_BF16, f"split, two launches {case} part {j}")
    # the two forms differ only by the fp32 summation order inside the shrink: a handful of last-bit differences
    differing = (ys[0] != y2).float().mean().item()
    assert differing < 5e-3, differing


def test_split_time_out_is_reported_and_survives_the_counter_reset():
    """A bounded in-launch wait that runs out must not pass silently.  Forced from the host: the row-block counters
    start at -1000 instead of zero, so the arrivals of the shrink workgroups never reach the target; every GEMM
    workgroup gives up after its 2^20 polls (about a quarter of a second) and the kernel ends normally.  The call's flag
    word says so, the per-device count says so after the arena has been reset, and check_split_timeouts raises once."""
    from katz_amd import _lib, ops

    say("lora_linear_split time-out")
    d = dev()
    M, N, K, R = 2048, 1280, 1280, 64
    lib = _lib.load()
    assert lib.kh_lora_linear_split_launches(M, N, K, R, 0, 0) == 1    # the shrink runs inside the launch
    g = torch.Generator().manual_seed(5)
    x, w = randn(g, M, K).to(d, BF), randn(g, N, K, std=0.03).to(d, BF)
    A, B = randn(g, R, K, std=0.05).to(d, BF), randn(g, N, R, std=0.05).to(d, BF)
    cs = torch.ones(R, device=d)
    t = torch.empty(M, R, dtype=BF, device=d)
    y = torch.empty(M, N, dtype=BF, device=d)
    torch.cuda.synchronize()
    ops.split_timeouts(d, clear=True)
    cnt = torch.full(((M + 127) // 128 + 1,), -1000, dtype=torch.int32, device=d)
    cnt[-1] = 0
    rc = lib.kh_lora_linear_split_bf16(x.data_ptr(), w.data_ptr(), None, A.data_ptr(), cs.data_ptr(), B.data_ptr(),
                                       t.data_ptr(), cnt.data_ptr(), None, y.data_ptr(), M, N, K, R, 0, 0,
                                       torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert int(cnt[-1]) == 1
    ops.split_counters_reset(d)                       # the next step's reset does not wipe the evidence
    assert ops.split_timeouts(d) >= 1
    with pytest.raises(ops.SplitTimeoutError):
        ops.check_split_timeouts(d)
    ops.check_split_timeouts(d)                       # cleared by the raising check


def test_cooperative_shrink_time_out_and_the_switch_for_a_second_stream():
    """The cooperative form (every GEMM workgroup delivers a piece of T, then waits for its row block's count): the
    same forced time-out as above ends the kernel normally and is reported; inside ops.side_branch() the form is not
    used (two such launches side by side could wait for each other's unscheduled workgroups) and the result is that
    of the two-launch form, bit for bit."""
    from katz_amd import _lib, ops

    say("cooperative shrink: time-out, side branch")
    d = dev()
    M, N, K, R, RU = 8192, 640, 640, 128, 96
    lib = _lib.load()
    fl = (RU // 16) << 16
    assert lib.kh_lora_linear_split_launches(M, N, K, R, 0, fl) == 1
    assert lib.kh_lora_linear_split_launches(M, N, K, R, 0, fl | (1 << 24)) == 2
    g = torch.Generator().manual_seed(6)
    x, w = randn(g, M, K).to(d, BF), randn(g, N, K, std=0.03).to(d, BF)
    A, B = randn(g, R, K, std=0.05), randn(g, N, R, std=0.05)
    A[RU:] = 0
    B[:, RU:] = 0
    A, B = A.to(d, BF), B.to(d, BF)
    cs = torch.ones(R, device=d)
    y_two = ops.lora_linear_split(x, w, None, A, cs, B, r_used=RU, two_launches=True)
    with ops.side_branch():
        y_side = ops.lora_linear_split(x, w, None, A, cs, B, r_used=RU)
    torch.cuda.synchronize()
    assert torch.equal(y_side, y_two)
    t = torch.empty(M, R, dtype=BF, device=d)
    y = torch.empty(M, N, dtype=BF, device=d)
    ops.split_timeouts(d, clear=True)
    cnt = torch.full(((M + 127) // 128 + 1,), -1000, dtype=torch.int32, device=d)
    cnt[-1] = 0
    torch.cuda.synchronize()
    rc = lib.kh_lora_linear_split_bf16(x.data_ptr(), w.data_ptr(), None, A.data_ptr(), cs.data_ptr(), B.data_ptr(),
                                       t.data_ptr(), cnt.data_ptr(), None, y.data_ptr(), M, N, K, R, 0, fl,
                                       torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert int(cnt[-1]) == 1
    # every piece of T was delivered all the same (the wait only ran out), so the result is still the right one
    assert (y != y_two).float().mean().item() < 5e-3
    assert ops.split_timeouts(d) >= 1
    with pytest.raises(ops.SplitTimeoutError):
        ops.check_split_timeouts(d)
    ops.check_split_timeouts(d)


def test_split_counters_after_a_reset_that_was_only_recorded():
    """A reset recorded into a HIP graph does not run at capture time.  Counters that eager calls dirtied before the
    capture must still be clear when later eager calls reach them: every slice shows exactly its own arrivals (a slice
    that was not cleared would show them on top of the old ones) and the results repeat bit for bit."""
    from katz_amd import ops

    say("split counters: recorded reset")
    d = dev()
    g = torch.Generator().manual_seed(77)
    M, N, K, R = 2048, 1280, 1280, 64
    x, w, b = randn(g, M, K).to(d, BF), randn(g, N, K, std=0.03).to(d, BF), randn(g, N).to(d, BF)
    A, B = randn(g, R, K, std=0.05).to(d, BF), randn(g, N, R, std=0.05).to(d, BF)
    cs = torch.full((R,), 0.7, device=d)
    call = lambda rows: ops.lora_linear_split(x[:rows], w, b, A, cs, B)
    assert ops._lib.load().kh_lora_linear_split_launches(M, N, K, R, 0, 0) == 1, "shape no longer runs as one launch"

    def burst(n_calls):
        outs, cnts = [], []
        for _ in range(n_calls):
            outs.append(call(M))
            cnts.append(ops.split_counters_last(d).clone())
        return outs, cnts

    ops.split_counters_reset(d)
    ref_outs, ref_cnts = burst(6)                      # dirties six slices
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):     # records a reset and ONE call: nothing of it runs now
            ops.split_counters_reset(d)
            y_graph = call(M)
    torch.cuda.current_stream().wait_stream(side)
    ops.split_counters_reset(d)                        # the next eager "step"
    outs, cnts = burst(6)                              # reaches the slices the capture's reset never cleared
    graph.replay()
    torch.cuda.synchronize()
    for o, c, rc in zip(outs, cnts, ref_cnts):
        assert torch.equal(c, rc), f"counters {c.tolist()} instead of {rc.tolist()}"
        assert int(c[-1]) == 0
        assert torch.equal(o, ref_outs[0])
    assert torch.equal(y_graph, ref_outs[0])
    ops.split_counters_reset(d)


@pytest.mark.parametrize("case", [
    # (M, N, K, R, r_used, geglu, n_split)
    (2048, 10240, 1280, 128, 96, True, 0),     # 256x320 tiles: the last 64-column stage runs two of its four steps
    (2048, 1280, 1280, 128, 96, False, 0),     # in-launch form on 128x128 tiles
    (2048, 3840, 1280, 128, 96, False, 1280),  # stacked q / k / v on 256x128 tiles
    (2048, 1280, 1280, 128, 48, False, 0),     # a whole stage of padding: one K tile fewer
    (1100, 1000, 640, 64, 16, False, 0),       # ragged shape on the 4-wave tiles (32-column stages)
    (8192, 640, 640, 128, 96, False, 0),       # 160-column tiles: the promise moves the shrink into the launch
    (8192, 640, 640, 128, 112, False, 0),      # ... and is accepted and not used beyond 96 columns
], ids=str)
def test_lora_linear_split_rank_padding_promise(case):
    """r_used: with the rank columns >= r_used of A_cat / B_cat zero (the padding of the packed adapters), the result is
    bit-identical with and without the promise, in one launch and in two (where the promise does not change the number
    of launches), and matches the oracle."""
    from katz_amd import ops

    from katz_amd.lora import interleave_geglu_rows

    M, N, K, R, r_used, geglu, n_split = case
    say("lora_linear_split r_used", case)
    d = dev()
    g = torch.Generator().manual_seed(M + N + K + R + r_used)
    parts = N // n_split if n_split else 1
    x, w = randn(g, M, K), randn(g, N, K, std=0.03)
    A, B = randn(g, parts, R, K, std=0.05), randn(g, N, R, std=0.05)
    A[:, r_used:] = 0
    B[:, r_used:] = 0
    xd, wd, Ad, Bd = x.to(d, BF), w.to(d, BF), A.reshape(parts * R, K).to(d, BF), B.to(d, BF)
    if geglu:
        wd, Bd = interleave_geglu_rows(wd), interleave_geglu_rows(Bd)
    cs = torch.full((parts * R,), 0.7, device=d)
    outs = {}
    for two in (False, True):
        for ru in (0, r_used):
            ops.split_counters_reset(d)
            outs[two, ru] = ops.lora_linear_split(xd, wd, None, Ad, cs, Bd, geglu=geglu, two_launches=two,
                                                  n_split=n_split, r_used=ru)
    torch.cuda.synchronize()
    launches = lambda ru: ops._lib.load().kh_lora_linear_split_launches(M, N, K, R, n_split, (1 if geglu else 0) | (ru // 16) << 16)
    for two in (False, True):
        if two or launches(0) == launches(r_used):
            assert torch.equal(outs[two, 0], outs[two, r_used]), f"two_launches={two}: the promise changed the result"
        else:   # the promise moved the shrink into the launch: another fp32 summation order, a few last-bit differences
            assert (outs[two, 0] != outs[two, r_used]).float().mean().item() < 5e-3
    xf, wf, Af, Bf = (t.float().cpu() for t in (x.to(BF), w.to(BF), A.to(BF), B.to(BF)))
    step = n_split if n_split else N
    for j in range(parts):
        rows = slice(j * step, (j + 1) * step)
        ref = O.lora_linear(xf, wf[rows], None, [(Af[j], Bf[rows], 0.7)])
        if geglu:
            ref = O.geglu(ref)
            assert_close_rel(outs[False, r_used], ref, REL_BF16, f"r_used {case}")
        else:
            assert_close_rel(outs[False, r_used][:, rows], ref, REL_BF16, f"r_used {case} part {j}")
    with pytest.raises(Exception):
        ops.lora_linear_split(xd, wd, None, Ad, cs, Bd, geglu=geglu, n_split=n_split, r_used=R + 16)
    ops.split_counters_reset(d)


# ------------------------------------------------------------------------------------------- batched merge
@pytest.mark.parametrize("op_dtype", [torch.float16, torch.bfloat16], ids=str)
def test_lora_merge_grouped(op_dtype):
    """kh_lora_merge_grouped_bf16: W_l += scale * s_l * up_l @ down_l for several layers of different shapes and ranks in
    one launch, against the oracle's merged weight (models/lora.py:409-425; Katz's patch_on_lora,
    pipeline_controlnet_sd_xl_katz.py:1743-1746); ragged sizes, rank 4 .. 128, fp16 (Katz's shared-memory dtype) and
    bf16 operands; a negative scale undoes the merge up to one rounding; weights not in the table are untouched."""
    from katz_amd import ops

    say("lora_merge_grouped", op_dtype)
    d = dev()
    g = torch.Generator().manual_seed(77)
    shapes = [(1280, 1280, 64), (640, 2048, 16), (10240, 1280, 128), (1280, 5120, 4), (200, 136, 24), (130, 60, 7), (64, 64, 64)]
    ws, ups, downs, scales = [], [], [], []
    for N, K, r in shapes:
        ws.append(randn(g, N, K, std=0.03).to(BF))
        ups.append(randn(g, N, r, std=0.2).to(op_dtype))
        downs.append(randn(g, r, K, std=0.2).to(op_dtype))
        scales.append(0.25 + 0.5 * len(scales))
    bystander = randn(g, 256, 256).to(d, BF)
    keep = bystander.clone()
    wd = [w.to(d).clone() for w in ws]
    v0 = [w._version for w in wd]
    ops.lora_merge_grouped(wd, [u.to(d) for u in ups], [x.to(d) for x in downs], scale=0.7, layer_scales=scales)
    torch.cuda.synchronize()
    assert all(w._version > v for w, v in zip(wd, v0))
    for w0, w1, u, x, s in zip(ws, wd, ups, downs, scales):
        ref = O.lora_merged_weight(w0.float(), [(x.float(), u.float(), 0.7 * s)])
        assert_close_rel(w1, ref, 4e-3, f"merged weight {tuple(w0.shape)}")     # one bf16 rounding of the sum
        assert (ref - w0.float()).abs().max() > 0.05
    assert torch.equal(bystander, keep)
    ops.lora_merge_grouped(wd, [u.to(d) for u in ups], [x.to(d) for x in downs], scale=-0.7, layer_scales=scales)
    torch.cuda.synchronize()
    for w0, w1, u, x, sc in zip(ws, wd, ups, downs, scales):
        # the merged weight was rounded to bf16 at ITS magnitude: undoing restores W up to that rounding
        merged_max = O.lora_merged_weight(w0.float(), [(x.float(), u.float(), 0.7 * sc)]).abs().max().item()
        assert (w1.float().cpu() - w0.float()).abs().max().item() <= 2.0 ** -7 * merged_max, tuple(w0.shape)
    with pytest.raises(ValueError):
        ops.lora_merge_grouped([wd[0], wd[0]], [ups[0].to(d)] * 2, [downs[0].to(d)] * 2)
    with pytest.raises(ValueError):
        ops.lora_merge_grouped([wd[0]], [ups[1].to(d)], [downs[0].to(d)])


def test_unet_fuse_lora_through_the_batched_merge():
    """UNet.fuse_lora / unfuse_lora on the GPU (safe_fusing=False: one merge launch per adapter over all linear layers)
    give the weights of the per-layer fp32 path (safe_fusing=True) and mark the same adapters as fused."""
    import katz_amd.layers as L
    from katz_amd.unet_2d_condition import UNet2DConditionModel, UNetConfig

    say("fuse_lora grouped")
    torch.manual_seed(0)
    unet = UNet2DConditionModel(UNetConfig.tiny()).to_runtime(dev(), BF)
    g = torch.Generator().manual_seed(5)
    lin = unet.lora_linears()
    for name, rank in (("a", 8), ("b", 4)):
        for m in lin.values():
            m.add_adapter(name, randn(g, rank, m.in_features, std=0.05).to(dev(), BF), randn(g, m.out_features, rank, std=0.05).to(dev(), BF), alpha=2.0 * rank)
    unet.set_adapters(["a", "b"], [0.8, 0.6])
    w0 = {n: m.weight.detach().clone() for n, m in lin.items()}
    unet.fuse_lora(0.5)
    fast = {n: m.weight.detach().clone() for n, m in lin.items()}
    assert all(m._fused == {"a": 0.5 * 0.8 * 2.0, "b": 0.5 * 0.6 * 2.0} for m in lin.values())
    assert all(m._packed is None for m in lin.values())          # fused adapters are not applied a second time
    unet.unfuse_lora()
    assert not any(m._fused for m in lin.values())
    for n, m in lin.items():
        assert_close_rel(m.weight, w0[n].float().cpu(), 2e-2, f"unfused {n}")   # two bf16 roundings of the merged weight
        with torch.no_grad():
            m.weight.copy_(w0[n])
    unet.fuse_lora(0.5, safe_fusing=True)
    for n, m in lin.items():
        assert_close_rel(fast[n], m.weight.float().cpu(), 8e-3, f"grouped vs per-layer fuse {n}")
        assert (m.weight.float() - w0[n].float()).abs().max() > 1e-3


# ------------------------------------------------------------------------------------------- conv_out + guidance + Euler
@pytest.mark.parametrize("Bl,H,W,C,f32", [(1, 128, 128, 320, False), (2, 16, 20, 64, False), (1, 9, 150, 48, True),
                                          (1, 32, 32, 64, True)], ids=str)
def test_conv_out_cfg_euler(Bl, H, W, C, f32):
    """kh_conv_out_cfg_euler_bf16 (the UNet's conv_out with guidance + Euler step + next input scaling as its epilogue)
    against the oracle: F.conv2d in fp32 rounded to the model dtype, then classifier_free_guidance and the scheduler's
    step formula; and against the two separate kernels of the product (conv3x3 + cfg_euler_step)."""
    from katz_amd import ops
    from oracle import euler as OE

    say("conv_out_cfg_euler", Bl, H, W, C, f32)
    d = dev()
    g = torch.Generator().manual_seed(Bl * 1000 + H + W + C)
    x = randn(g, 2 * Bl, C, H, W).to(BF)
    w = randn(g, 4, C, 3, 3, std=(9 * C) ** -0.5).to(BF)
    b = randn(g, 4, std=0.1).to(BF)
    lat = (randn(g, Bl, 4, H, W) * 3).to(BF)
    sigma, sigma_next, gs = 4.2, 3.1, 7.5
    coef = torch.tensor([sigma, sigma_next, (sigma_next ** 2 + 1) ** 0.5], dtype=torch.float32)
    cl = lambda t: t.to(d).contiguous(memory_format=torch.channels_last)
    lat_d = cl(lat.float() if f32 else lat)
    nxt = torch.empty(2 * Bl, 4, H, W, dtype=BF, device=d).contiguous(memory_format=torch.channels_last)
    noise = torch.empty_like(nxt)
    out = ops.conv_out_cfg_euler(cl(x), ops.pack_conv3x3_weight(w.to(d)), b.to(d), lat_d, coef.to(d), gs,
                                 model_input_next=nxt, noise_pred_out=noise)
    torch.cuda.synchronize()
    # oracle
    ref_noise = bf16_round(torch.nn.functional.conv2d(x.float(), w.float(), b.float(), padding=1))
    assert_close_rel(noise, ref_noise, REL_BF16, "conv_out noise")
    u, t = noise.float().cpu()[:Bl], noise.float().cpu()[Bl:]          # the kernel's own rounded noise: exact arithmetic after it
    eps = u + gs * (t - u)
    xin = lat.float()
    x0 = xin - sigma * eps
    want = xin + ((xin - x0) / sigma) * (coef[1] - coef[0])
    if not f32:
        want = bf16_round(want)
    assert out.dtype == (torch.float32 if f32 else BF)
    assert (out.float().cpu() - want).abs().max().item() <= 1e-5 * want.abs().max().item() + (0 if f32 else 2 ** -8 * want.abs().max().item())
    want_next = bf16_round(want / coef[2])
    assert_close_rel(nxt[:Bl], want_next, 1e-2, "next input")
    assert torch.equal(nxt[:Bl], nxt[Bl:])
    # the product's two separate kernels on the same inputs
    from katz_amd.layers import Conv3x3
    conv = Conv3x3(C, 4)
    with torch.no_grad():
        conv.weight.copy_(w.float()); conv.bias.copy_(b.float())
    conv = conv.to(d, BF)
    with torch.no_grad():
        e2 = conv(cl(x))
    out2 = ops.cfg_euler_step(e2, lat_d, coef.to(d), gs)
    assert_close_rel(noise, e2.float().cpu(), 1e-2, "fused conv vs conv kernel")
    assert cosine(out, out2) >= 0.99999


# ------------------------------------------------------------------------------------------- more than 128 rank columns
@pytest.mark.parametrize("geglu", [False, True], ids=["linear", "geglu"])
def test_lora_linear_with_more_than_128_rank_columns(geglu):
    """Three rank-64 adapters and one rank-160 adapter active at once (peft has no limit on the sum of ranks): the
    layer applies the first 128 rank columns in the fused launch and the rest pack by pack; against the oracle."""
    from katz_amd.layers import LoRALinear

    say("lora_linear wide rank", geglu)
    d = dev()
    g = torch.Generator().manual_seed(31)
    K, N, M = 640, 1280, 300
    lin = LoRALinear(K, N, geglu=geglu)
    with torch.no_grad():
        lin.weight.copy_(randn(g, N, K, std=0.03).to(BF).float()); lin.bias.copy_(randn(g, N, std=0.1).to(BF).float())
    w, b = lin.weight.detach().clone(), lin.bias.detach().clone()
    lin = lin.to(d, BF)
    specs = [("a", 64, 0.8), ("b", 64, 0.6), ("c", 64, 1.1), ("d", 160, 0.4)]
    ads = []
    for name, r, wt in specs:
        A, B = randn(g, r, K, std=0.05).to(BF).float(), randn(g, N, r, std=0.05).to(BF).float()
        lin.add_adapter(name, A, B, alpha=float(r))
        ads.append((A, B, wt))
    lin.set_active([s[0] for s in specs], [s[2] for s in specs])
    assert len(lin._packed.overflow) == 2      # 352 rank columns: 128 + 128 + 96
    x = randn(g, M, K).to(BF)
    res = None if geglu else randn(g, M, N).to(BF)
    with torch.no_grad():
        y = lin(x.to(d), residual=None if res is None else res.to(d))
        torch.cuda.synchronize()
    ref = O.lora_linear(x.float(), w, b, ads, residual=None if res is None else res.float())
    if geglu:
        ref = O.geglu(ref)
    # every extra pack rounds y to bf16 once more (three roundings here, then the activation): 3e-2 instead of 2e-2
    assert_close_rel(y, ref, 3e-2 if geglu else REL_BF16, "wide-rank lora linear")
    lin.set_active(["a"], [1.0])
    assert not lin._packed.overflow
