"""LayerNorm folded into the LoRA linear (kh_lora_linear_norm_bf16) against the oracle's LayerNorm followed by its LoRA
linear, and the row statistics a producer leaves for it against plain sums -- at the SDXL shapes that reach each of the
GEMM kernels (128x128 with and without the shrink inside the launch, 256x128 stacked q/k/v, 64/128x160, 256x320 with
GEGLU) and on ragged shapes.

Tolerance: the parity contract's 2e-2 * (|ref| + rms(ref)) for bf16 kernels; the statistics 1e-3 relative (fp32 sums
of bf16-rounded outputs in another order).
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


def _stats_of(y):
    y = y.float()
    return y.sum(-1), (y * y).sum(-1)


@pytest.mark.parametrize("M,N,K,R,res", [
    (2048, 1280, 1280, 0, True),     # 128x128, 8 waves
    (2048, 1280, 1280, 128, True),   # shrink inside the launch
    (2048, 1280, 5120, 0, True),     # 64x160, K split over the waves
    (2048, 1280, 5120, 128, True),
    (8192, 640, 640, 0, True),       # 128x160
    (8192, 640, 640, 64, False),
    (8192, 640, 2560, 128, True),
    (300, 384, 128, 0, True),        # ragged
    (300, 2048, 192, 64, False),     # 16 column tiles
])
def test_row_statistics_of_the_output(M, N, K, R, res):
    from katz_amd import ops
    say("row statistics", M, N, K, R, res)
    g = torch.Generator().manual_seed(M + N + K + R)
    x, w, b = randn(g, M, K), randn(g, N, K, std=0.03), randn(g, N, std=0.1)
    r = randn(g, M, N) if res else None
    d = dev()
    a = s = bc = None
    ads = []
    if R:
        A, B = randn(g, R, K, std=0.05), randn(g, N, R, std=0.05)
        a, bc = A.to(d, BF), B.to(d, BF)
        s = torch.full((R,), 0.7, device=d)
        ads = [(A, B, 0.7)]
    st = ops.row_stats_buffer(M, d)
    st.fill_(float("nan"))   # every slot must be written
    y = ops.lora_linear_norm(x.to(d, BF), w.to(d, BF), b.to(d, BF), a, s, bc, residual=None if r is None else r.to(d, BF),
                             stats_out=st)
    torch.cuda.synchronize()
    ref = O.lora_linear(x, w, b, ads, residual=r)
    assert_close_rel(y, ref, 2e-2, "linear with stats_out")
    # bit-equal to the same layer without the statistics
    if R:
        y0 = ops.lora_linear_split(x.to(d, BF), w.to(d, BF), b.to(d, BF), a, s, bc, residual=None if r is None else r.to(d, BF))
    else:
        y0 = ops.lora_linear(x.to(d, BF), w.to(d, BF), b.to(d, BF), residual=None if r is None else r.to(d, BF))
    assert torch.equal(y, y0)
    s1, s2 = _stats_of(y)
    got = st.double().sum(0).cpu()
    assert torch.isfinite(got).all()
    assert torch.allclose(got[:, 0], s1.double().cpu(), rtol=1e-3, atol=1e-2 * float(s2.max().sqrt()))
    assert torch.allclose(got[:, 1], s2.double().cpu(), rtol=1e-3)


def _fold_case(M, N, K, R, seed, n_split=0, shift=0.5):
    g = torch.Generator().manual_seed(seed)
    h = randn(g, M, K) * 1.5 + shift             # rows with a mean: the mean term must matter
    h = bf16_round(h)
    gamma = bf16_round(1.0 + 0.2 * torch.randn(K, generator=g))
    beta = randn(g, K, std=0.2)
    w = randn(g, N, K, std=0.03)
    b = randn(g, N, std=0.1)
    groups = N // n_split if n_split else 1
    A = randn(g, groups * R, K, std=0.05) if R else None
    B = randn(g, N, R, std=0.05) if R else None
    return h, gamma, beta, w, b, A, B


def _ref_fold(h, gamma, beta, w, b, A, B, scale, n_split=0, geglu=False, exact=False):
    """exact: float64 throughout.  Otherwise rounded to bf16 where the reference's half-precision modules round: the
    normalised rows, the projection, the activation."""
    rnd = (lambda t: t) if exact else bf16_round
    if exact:
        h, gamma, beta, w, b = h.double(), gamma.double(), beta.double(), w.double(), b.double()
        A, B = (None, None) if A is None else (A.double(), B.double())
    x = rnd(O.layer_norm(h, gamma, beta, 1e-5))
    N = w.shape[0]
    if A is None:
        y = O.lora_linear(x, w, b)
    elif not n_split:
        y = O.lora_linear(x, w, b, [(A, B, scale)])
    else:
        R = B.shape[1]
        ys = []
        for j in range(N // n_split):
            sl = slice(j * n_split, (j + 1) * n_split)
            ys.append(O.lora_linear(x, w[sl], None if b is None else b[sl], [(A[j * R:(j + 1) * R], B[sl], scale)]))
        y = torch.cat(ys, dim=-1)
    if not geglu:
        return y
    v, gate = rnd(y).chunk(2, dim=-1)
    return v * rnd(O.gelu(gate))


def _rms_err(got, exact):
    got, exact = got.detach().double().cpu(), exact.double()
    return float((got - exact).pow(2).mean().sqrt() / exact.pow(2).mean().sqrt())


def _stats_from(h, d):
    """What a producer would have left for the rows of h: here from torch, spread over three slots."""
    from katz_amd import ops
    M, K = h.shape
    st = torch.zeros((ops.LN_SLOTS, M, 2), dtype=torch.float32)
    cuts = [0, K // 3 // 8 * 8, K // 2, K]
    for j in range(3):
        part = h[:, cuts[j]:cuts[j + 1]].float()
        st[j, :, 0] = part.sum(-1)
        st[j, :, 1] = (part * part).sum(-1)
    return st.to(d)


@pytest.mark.parametrize("M,N,K,R,n_split,geglu", [
    (2048, 1280, 1280, 0, 0, False),      # attn2.to_q, no adapters: 128x128, 8 waves
    (2048, 1280, 1280, 128, 0, False),    # with adapters: shrink inside the launch
    (2048, 3840, 1280, 0, 0, False),      # stacked q/k/v: 256x128
    (2048, 3840, 1280, 128, 1280, False),
    (2048, 10240, 1280, 0, 0, True),      # GEGLU projection: 256x320
    (2048, 10240, 1280, 128, 0, True),
    (8192, 640, 640, 0, 0, False),        # 128x160
    (8192, 640, 640, 64, 0, False),
    (8192, 1920, 640, 128, 640, False),   # stacked q/k/v at 64x64 resolution
    (8192, 5120, 640, 128, 0, True),
    (300, 384, 128, 0, 0, False),         # ragged
    (300, 384, 128, 64, 0, False),
    (77, 256, 64, 0, 0, True),
])
def test_layer_norm_folded_into_the_linear(M, N, K, R, n_split, geglu):
    from katz_amd import ops
    from katz_amd.lora import fold_layer_norm, interleave_geglu_rows
    say("folded LayerNorm", M, N, K, R, n_split, geglu)
    d = dev()
    h, gamma, beta, w, b, A, B = _fold_case(M, N, K, R, seed=M + N + K + R, n_split=n_split)
    scale = 0.8
    ref = _ref_fold(h, gamma, beta, w, b, A, B, scale, n_split, geglu)
    wk, bk, Bk = w, b, B
    if geglu:
        wk, bk = interleave_geglu_rows(w), interleave_geglu_rows(b)
        Bk = interleave_geglu_rows(B) if B is not None else None
    wp, c1, c2, ap, ca1, ca2 = fold_layer_norm(wk.to(d, BF), bk.to(d, BF), gamma.to(d, BF), beta.to(d, BF),
                                               None if A is None else A.to(d, BF))
    st = _stats_from(h, d)
    s = None if A is None else torch.full((A.shape[0],), scale, device=d)
    y = ops.lora_linear_norm(h.to(d, BF), wp, None, ap, s, None if Bk is None else Bk.to(d, BF).contiguous(), geglu=geglu,
                             n_split=n_split, ln=(st, c1, c2, ca1, ca2, 1e-5))
    torch.cuda.synchronize()
    exact = _ref_fold(h, gamma, beta, w, b, A, B, scale, n_split, geglu, exact=True)
    e_ref, e_got = _rms_err(bf16_round(ref), exact), _rms_err(y, exact)
    say(f"  rms error against float64: reference's rounding {e_ref:.2e}, folded kernel {e_got:.2e}")
    assert e_got <= 1.25 * e_ref + 1e-4, "the fold is less accurate than LayerNorm -> bf16 -> linear"
    assert_close_rel(y, exact.float(), 4e-2 if geglu else 2e-2, "folded LayerNorm + linear")
    if R:   # the two-launch form gives the same numbers up to the shrink's summation order
        y2 = ops.lora_linear_norm(h.to(d, BF), wp, None, ap, s, Bk.to(d, BF).contiguous(), geglu=geglu, n_split=n_split,
                                  two_launches=True, ln=(st, c1, c2, ca1, ca2, 1e-5))
        assert _rms_err(y2, exact) <= 1.25 * e_ref + 1e-4
        assert_close_rel(y2, exact.float(), 4e-2 if geglu else 2e-2, "folded LayerNorm + linear, two launches")


@pytest.mark.parametrize("M,N,K,n_split,res,stats", [
    (8192, 640, 640, 0, False, False),      # a folded LayerNorm in front
    (8192, 640, 2560, 0, True, True),       # ff.net.2: residual, statistics for the next block's norm1
    (8192, 640, 640, 0, True, True),        # to_out
    (8000, 640, 640, 0, False, True),       # ragged rows
])
def test_cooperative_shrink_with_fold_and_statistics(M, N, K, n_split, res, stats):
    """Ranks 64 + 32 in 128 packed columns (r_used = 96) on the layers whose 128 x 160 tiles fill the chip: every GEMM
    workgroup first computes a 32 x 96 piece of T, with the folded LayerNorm's correction where there is one.  Against
    float64, against the two-launch form, and the row statistics of the result."""
    from katz_amd import ops
    from katz_amd.lora import fold_layer_norm
    say("cooperative shrink + fold / statistics", M, N, K, n_split, res, stats)
    d = dev()
    R, RU = 128, 96
    fold = not res
    h, gamma, beta, w, b, A, B = _fold_case(M, N, K, R, seed=M + N + K + 96, n_split=n_split)
    parts = N // n_split if n_split else 1
    for j in range(parts):
        A[j * R + RU:(j + 1) * R] = 0
    B[:, RU:] = 0
    scale = 0.8
    assert ops._lib.load().kh_lora_linear_split_launches(M, N, K, R, n_split, (RU // 16) << 16) == 1
    assert ops._lib.load().kh_lora_linear_split_launches(M, N, K, R, n_split, 0) == 2
    s = torch.full((A.shape[0],), scale, device=d)
    r = None
    if res:
        g = torch.Generator().manual_seed(M + 1)
        r = bf16_round(randn(g, M, N))
    st_out = None
    if stats:
        st_out = ops.row_stats_buffer(M, d)
        st_out.fill_(float("nan"))
    ops.split_counters_reset(d)
    if fold:
        wp, c1, c2, ap, ca1, ca2 = fold_layer_norm(w.to(d, BF), b.to(d, BF), gamma.to(d, BF), beta.to(d, BF), A.to(d, BF))
        ln = (_stats_from(h, d), c1, c2, ca1, ca2, 1e-5)
        run = lambda **kw: ops.lora_linear_norm(h.to(d, BF), wp, None, ap, s, B.to(d, BF), n_split=n_split, r_used=RU, ln=ln,
                                                stats_out=st_out, **kw)
        exact = _ref_fold(h, gamma, beta, w, b, A, B, scale, n_split, exact=True)
        e_ref = _rms_err(bf16_round(_ref_fold(h, gamma, beta, w, b, A, B, scale, n_split)), exact)
    else:
        run = lambda **kw: ops.lora_linear_norm(h.to(d, BF), w.to(d, BF), b.to(d, BF), A.to(d, BF), s, B.to(d, BF),
                                                residual=r.to(d, BF), n_split=n_split, r_used=RU, stats_out=st_out, **kw)
        exact = O.lora_linear(h.double(), w.double(), b.double(), [(A.double(), B.double(), scale)], residual=r.double())
        e_ref = 0.0
    y = run()
    flag = ops.split_counters_last(d)[-1:].clone()
    got = None if st_out is None else st_out.double().sum(0).cpu()
    y2 = run(two_launches=True)
    torch.cuda.synchronize()
    assert int(flag) == 0
    assert_close_rel(y, exact.float(), 2e-2, "cooperative shrink")
    if fold:
        assert _rms_err(y, exact) <= 1.25 * e_ref + 1e-4
    assert (y != y2).float().mean().item() < 5e-3          # the shrink's fp32 summation order differs
    if stats:
        s1, s2 = _stats_of(y)
        assert torch.isfinite(got).all()
        assert torch.allclose(got[:, 0], s1.double().cpu(), rtol=1e-3, atol=1e-2 * float(s2.max().sqrt()))
        assert torch.allclose(got[:, 1], s2.double().cpu(), rtol=1e-3)
    ops.check_split_timeouts(d)


def test_producer_feeds_consumer():
    """to_out (residual, statistics out) -> norm -> to_q with the norm folded: against the unfused chain."""
    from katz_amd import ops
    from katz_amd.lora import fold_layer_norm
    d = dev()
    g = torch.Generator().manual_seed(5)
    M, D = 2048, 1280
    a, res = randn(g, M, D), randn(g, M, D)
    w_out, b_out = randn(g, D, D, std=0.03), randn(g, D, std=0.1)
    gamma, beta = bf16_round(1.0 + 0.2 * torch.randn(D, generator=g)), randn(g, D, std=0.2)
    w_q = randn(g, D, D, std=0.03)
    st = ops.row_stats_buffer(M, d)
    h = ops.lora_linear_norm(a.to(d, BF), w_out.to(d, BF), b_out.to(d, BF), residual=res.to(d, BF), stats_out=st)
    wp, c1, c2, _, _, _ = fold_layer_norm(w_q.to(d, BF), None, gamma.to(d, BF), beta.to(d, BF))
    q = ops.lora_linear_norm(h, wp, None, ln=(st, c1, c2, None, None, 1e-5))
    n = ops.layer_norm(h, gamma.to(d, BF), beta.to(d, BF), 1e-5)
    q0 = ops.lora_linear(n, w_q.to(d, BF), None)
    torch.cuda.synchronize()
    assert_close_rel(q, q0, 2e-2, "folded chain against LayerNorm kernel + linear")
    ref = O.lora_linear(bf16_round(O.layer_norm(h.float().cpu(), gamma, beta, 1e-5)), w_q, None)
    assert_close_rel(q, ref, 2e-2, "folded chain against the oracle")


def test_transformer_with_and_without_the_fold(monkeypatch):
    """A transformer of SDXL's widths (proj_in -> two blocks -> proj_out) with adapters on every linear: the folded
    path against the same modules with every LayerNorm as a kernel of its own, and both against the oracle's blocks."""
    import katz_amd.layers as L
    from helpers import cosine, random_lora, round_module_to_bf16_
    from oracle import blocks as OB

    say("transformer, LayerNorm fold on / off")
    d = dev()
    torch.manual_seed(3)
    dim, heads, ctx_dim, H = 640, 10, 2048, 32
    oracle = OB.Transformer2DModel(heads, 64, dim, num_layers=2, cross_attention_dim=ctx_dim, use_linear_projection=True)
    for m in oracle.modules():   # LayerNorms with a weight and a bias that matter
        if isinstance(m, torch.nn.LayerNorm):
            torch.nn.init.normal_(m.weight, 1.0, 0.2); torch.nn.init.normal_(m.bias, 0.0, 0.2)
    round_module_to_bf16_(oracle)
    linears = {n: m for n, m in oracle.named_modules() if isinstance(m, OB.OracleLoRALinear)}
    lora = random_lora(linears, 16, seed=4, std=0.05)
    for n, m in linears.items():
        m.add_adapter("a", lora[n][0], lora[n][1], weight=0.9)
        m.active = ["a"]
    prod = L.Transformer2DModel(heads, 64, dim, num_layers=2, cross_attention_dim=ctx_dim)
    prod.load_state_dict(oracle.state_dict(), strict=True)
    prod = prod.to(d, BF)
    for name, m in prod.named_modules():
        if isinstance(m, L.LoRALinear) and name in lora:
            down, up = lora[name]
            m.add_adapter("a", down.to(d, BF), up.to(d, BF), weight=0.9)
            m.set_active(["a"])
    g = torch.Generator().manual_seed(6)
    x = bf16_round(torch.randn(2, dim, H, H, generator=g) * 1.5 + 0.3)
    ctx = bf16_round(torch.randn(2, 77, ctx_dim, generator=g))
    xd = x.to(d, BF).contiguous(memory_format=torch.channels_last)
    with torch.no_grad():
        ref = oracle(x, ctx)
        assert L.LN_FOLD
        from katz_amd import ops
        ops.CALL_LOG = []
        y1 = prod(xd, ctx.to(d, BF))
        log1, ops.CALL_LOG = ops.CALL_LOG, None
        monkeypatch.setattr(L, "LN_FOLD", False)
        ops.CALL_LOG = []
        y0 = prod(xd, ctx.to(d, BF))
        log0, ops.CALL_LOG = ops.CALL_LOG, None
    torch.cuda.synchronize()
    assert sum(1 for e in log0 if e[0] == "layer_norm") == 6 and not any(e[0] == "layer_norm" for e in log1)
    # (a folded launch logs two more fields: whether it folds a norm in front, whether it leaves row statistics)
    assert [e[:7] for e in log0 if e[0] != "layer_norm"] == [e[:7] for e in log1], "the same GEMM launches either way"
    c1, c0, c10 = cosine(y1, ref), cosine(y0, ref), cosine(y1, y0)
    say(f"  cosine against the oracle: folded {c1:.6f}, separate norms {c0:.6f}; folded against separate {c10:.6f}")
    assert c1 >= 0.9995 and c0 >= 0.9995 and c10 >= 0.9995
    assert_close_rel(y1, ref, 6e-2, "transformer with folded LayerNorms")
