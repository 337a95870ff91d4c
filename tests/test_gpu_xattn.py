"""A cross-attention's query projection with the attention inside its epilogue (kh_lora_linear_xattn_bf16) against the
oracle's LoRA linear (behind its LayerNorm where one is folded) followed by the oracle's attention, and against the
library's own two calls (projection, then kh_attention_bf16).

Tolerance: two bf16 kernels of the parity contract's 2e-2 * (|ref| + rms(ref)) each in a row (the rounding of q moves
the softmax): 4e-2 elementwise, as for the other two-stage chains (projection + GEGLU).  Against the library's two-call
form the results differ by rounding only (one softmax pass over all keys instead of a running maximum over 64-key
tiles): the same tolerance, and the rms error against the float64 result may not be worse than the two-call form's.
"""
import pytest
import torch

from helpers import assert_close_rel, bf16_round
from oracle import ops as O

pytestmark = pytest.mark.gpu
BF = torch.bfloat16
CHAIN_TOL = 4e-2


def dev():
    return torch.device("cuda:0")


def randn(g, *shape, std=1.0):
    return bf16_round(torch.randn(*shape, generator=g) * std)


def say(*a):
    print(*a, flush=True)


def _rms_err(got, exact):
    got, exact = got.detach().double().cpu(), exact.double()
    return float((got - exact).pow(2).mean().sqrt() / exact.pow(2).mean().sqrt())


def _case(B, T, heads, K, S, R, seed):
    g = torch.Generator().manual_seed(seed)
    N = heads * 64
    x = randn(g, B, T, K)
    w = randn(g, N, K, std=K ** -0.5)
    k, v = randn(g, B, S, N), randn(g, B, S, N)
    A = Bm = None
    if R:
        A, Bm = randn(g, R, K, std=0.05), randn(g, N, R, std=0.05)
    return x, w, k, v, A, Bm


def _ref(x, w, k, v, heads, A, Bm, scale, ln=None, exact=False):
    rnd = (lambda t: t) if exact else bf16_round
    if exact:
        x, w, k, v = x.double(), w.double(), k.double(), v.double()
        A, Bm = (None, None) if A is None else (A.double(), Bm.double())
    h = x
    if ln is not None:
        gamma, beta = ln
        if exact:
            gamma, beta = gamma.double(), beta.double()
        h = rnd(O.layer_norm(x, gamma, beta, 1e-5))
    q = rnd(O.lora_linear(h, w, None, () if A is None else [(A, Bm, scale)]))
    return O.attention(q, k, v, heads)


@pytest.mark.parametrize("B,T,heads,K,S,R,counters", [
    (2, 1024, 20, 1280, 77, 0, True),      # SDXL's attn2 at 32x32, no adapters
    (2, 1024, 20, 1280, 77, 128, True),    # with adapters: the shrink runs inside the launch
    (2, 1024, 20, 1280, 77, 64, False),    # two launches: shrink, then projection + attention
    (1, 1024, 20, 1280, 77, 128, True),    # batch 1
    (4, 256, 4, 192, 96, 0, True),         # every key slot used
    (3, 128, 2, 64, 1, 64, True),          # one key: softmax is 1, o = v
    (2, 384, 6, 320, 33, 0, True),
])
def test_query_projection_with_attention(B, T, heads, K, S, R, counters):
    from katz_amd import ops
    say("xattn", B, T, heads, K, S, R, counters)
    d = dev()
    x, w, k, v, A, Bm = _case(B, T, heads, K, S, R, seed=B * 1000 + T + heads + K + S + R)
    assert ops.lora_linear_xattn_ok(B * T, heads * 64, K, R, T, S, heads)
    scale = 0.6
    a = s = bc = None
    if R:
        a, bc = A.to(d, BF), Bm.to(d, BF)
        s = torch.full((R,), scale, device=d)
    kd, vd = k.to(d, BF), v.to(d, BF)
    o = ops.lora_linear_xattn(x.to(d, BF), w.to(d, BF), kd, vd, heads, a_cat=a, col_scale=s, b_cat=bc,
                              two_launches=not counters)
    # the same through two calls
    if R:
        q2 = ops.lora_linear_split(x.to(d, BF), w.to(d, BF), None, a, s, bc)
    else:
        q2 = ops.lora_linear(x.to(d, BF), w.to(d, BF), None)
    o2 = ops.attention(q2, kd, vd, heads)
    torch.cuda.synchronize()
    assert o.shape == (B, T, heads * 64)
    ref = _ref(x, w, k, v, heads, A, Bm, scale)
    exact = _ref(x, w, k, v, heads, A, Bm, scale, exact=True)
    e1, e2 = _rms_err(o, exact), _rms_err(o2, exact)
    say(f"  rms error against float64: one launch {e1:.2e}, projection + attention {e2:.2e}")
    assert_close_rel(o, ref, CHAIN_TOL, "projection + attention in one launch against the oracle")
    assert_close_rel(o, o2.float().cpu(), CHAIN_TOL, "one launch against the library's two calls")
    assert e1 <= 1.25 * e2 + 1e-4
    if S == 1:
        assert torch.equal(o.cpu(), vd.cpu().expand(B, T, heads * 64)), "one key: the output is that key's value"


def test_kv_as_views_of_one_projection():
    """k and v as column slices of one [B,S,2N] buffer (the context projected for k and v side by side)."""
    from katz_amd import ops
    say("xattn, strided k / v")
    d = dev()
    B, T, heads, K, S = 2, 512, 10, 640, 77
    N = heads * 64
    x, w, _, _, _, _ = _case(B, T, heads, K, S, 0, seed=11)
    g = torch.Generator().manual_seed(12)
    kv = randn(g, B, S, 2 * N)
    kvd = kv.to(d, BF)
    kd, vd = kvd.split(N, dim=-1)
    o = ops.lora_linear_xattn(x.to(d, BF), w.to(d, BF), kd, vd, heads)
    torch.cuda.synchronize()
    k, v = kv.split(N, dim=-1)
    ref = _ref(x, w, k.contiguous(), v.contiguous(), heads, None, None, 1.0)
    assert_close_rel(o, ref, CHAIN_TOL, "strided k / v")


@pytest.mark.parametrize("R", [0, 128])
def test_folded_layer_norm_in_front(R):
    """norm2 -> attn2.to_q -> attention: the norm folded into the projection (row statistics from the producer)."""
    from katz_amd import ops
    from katz_amd.lora import fold_layer_norm
    say("xattn behind a folded LayerNorm", R)
    d = dev()
    B, T, heads, K, S = 2, 1024, 20, 1280, 77
    M = B * T
    x, w, k, v, A, Bm = _case(B, T, heads, K, S, R, seed=21 + R)
    g = torch.Generator().manual_seed(22)
    x = bf16_round(x * 2.0 + 0.5)
    gamma, beta = bf16_round(1.0 + 0.2 * torch.randn(K, generator=g)), randn(g, K, std=0.2)
    st = torch.zeros((ops.LN_SLOTS, M, 2), dtype=torch.float32)
    xf = x.reshape(M, K).float()
    st[0, :, 0], st[0, :, 1] = xf.sum(-1), (xf * xf).sum(-1)
    st = st.to(d)
    scale = 0.8
    wp, c1, c2, ap, ca1, ca2 = fold_layer_norm(w.to(d, BF), None, gamma.to(d, BF), beta.to(d, BF), None if A is None else A.to(d, BF))
    s = None if A is None else torch.full((R,), scale, device=d)
    o = ops.lora_linear_xattn(x.to(d, BF), wp, k.to(d, BF), v.to(d, BF), heads, a_cat=ap, col_scale=s,
                              b_cat=None if Bm is None else Bm.to(d, BF), ln=(st, c1, c2, ca1, ca2, 1e-5))
    torch.cuda.synchronize()
    ref = _ref(x, w, k, v, heads, A, Bm, scale, ln=(gamma, beta))
    exact = _ref(x, w, k, v, heads, A, Bm, scale, ln=(gamma, beta), exact=True)
    say(f"  rms error against float64: {_rms_err(o, exact):.2e} (reference's rounding {_rms_err(bf16_round(ref), exact):.2e})")
    assert_close_rel(o, ref, CHAIN_TOL, "folded LayerNorm + projection + attention")


def test_shapes_that_are_not_taken():
    from katz_amd import _lib, ops
    say("xattn, refused shapes")
    d = dev()
    assert not ops.lora_linear_xattn_ok(2048, 1280, 1280, 0, 1024, 97, 20)      # too many keys
    assert not ops.lora_linear_xattn_ok(2 * 4096, 640, 640, 0, 4096, 77, 10)    # more than one round of tiles
    assert not ops.lora_linear_xattn_ok(2 * 1000, 1280, 1280, 0, 1000, 77, 20)  # ragged query count
    assert not ops.lora_linear_xattn_ok(2048, 1280, 1280, 32, 1024, 77, 20)     # rank padding of 32
    x = torch.zeros((2, 1000, 1280), dtype=BF, device=d)
    w = torch.zeros((1280, 1280), dtype=BF, device=d)
    kv = torch.zeros((2, 77, 1280), dtype=BF, device=d)
    with pytest.raises(_lib.KatzHipError):
        ops.lora_linear_xattn(x, w, kv, kv, 20)


@pytest.mark.parametrize("adapters", [False, True])
def test_transformer_with_and_without_the_fused_attention(monkeypatch, adapters):
    """A transformer of SDXL's 32x32 level (width 1280, 20 heads, two blocks): the attention processor with the
    cross-attention inside the query projection's launch against the same modules running projection and attention
    kernel one after the other, and both against the oracle's blocks."""
    import katz_amd.layers as L
    from helpers import cosine, random_lora, round_module_to_bf16_
    from katz_amd import ops
    from oracle import blocks as OB

    say("transformer, attention inside the query projection on / off; adapters:", adapters)
    d = dev()
    torch.manual_seed(3)
    dim, heads, ctx_dim, H = 1280, 20, 2048, 32
    oracle = OB.Transformer2DModel(heads, 64, dim, num_layers=2, cross_attention_dim=ctx_dim, use_linear_projection=True)
    for m in oracle.modules():
        if isinstance(m, torch.nn.LayerNorm):
            torch.nn.init.normal_(m.weight, 1.0, 0.2); torch.nn.init.normal_(m.bias, 0.0, 0.2)
    round_module_to_bf16_(oracle)
    prod = L.Transformer2DModel(heads, 64, dim, num_layers=2, cross_attention_dim=ctx_dim)
    prod.load_state_dict(oracle.state_dict(), strict=True)
    prod = prod.to(d, BF)
    if adapters:
        linears = {n: m for n, m in oracle.named_modules() if isinstance(m, OB.OracleLoRALinear)}
        lora = random_lora(linears, 16, seed=4, std=0.05)
        for n, m in linears.items():
            m.add_adapter("a", lora[n][0], lora[n][1], weight=0.9)
            m.active = ["a"]
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
        assert L.XATTN_FUSE
        ops.CALL_LOG = []
        y1 = prod(xd, ctx.to(d, BF))
        log1, ops.CALL_LOG = ops.CALL_LOG, None
        monkeypatch.setattr(L, "XATTN_FUSE", False)
        ops.CALL_LOG = []
        y0 = prod(xd, ctx.to(d, BF))
        log0, ops.CALL_LOG = ops.CALL_LOG, None
    torch.cuda.synchronize()
    n1 = sum(1 for e in log1 if e[0] == "lora_linear_xattn")
    assert n1 == 2 and not any(e[0] == "lora_linear_xattn" for e in log0), "one fused launch per block"
    assert sum(1 for e in log0 if e[0] == "attention") - sum(1 for e in log1 if e[0] == "attention") == 2
    assert len(log0) - len(log1) == 2, "two launches fewer"
    c1, c0, c10 = cosine(y1, ref), cosine(y0, ref), cosine(y1, y0)
    say(f"  cosine against the oracle: fused {c1:.6f}, separate {c0:.6f}; fused against separate {c10:.6f}")
    assert c1 >= 0.9995 and c0 >= 0.9995 and c10 >= 0.9995
    assert_close_rel(y1, ref, 6e-2, "transformer with the attention inside the query projection")
