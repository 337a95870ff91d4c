"""Pins of oracle/ops.py: library routines, identities and brute force -- no formula is retyped here."""
import math

import torch
import torch.nn.functional as F

from oracle import ops as O


def test_lora_linear_brute_force_fp64():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(3, 5, generator=g, dtype=torch.float64)
    W = torch.randn(4, 5, generator=g, dtype=torch.float64)
    b = torch.randn(4, generator=g, dtype=torch.float64)
    ads = [(torch.randn(2, 5, generator=g, dtype=torch.float64), torch.randn(4, 2, generator=g, dtype=torch.float64), 0.7),
           (torch.randn(3, 5, generator=g, dtype=torch.float64), torch.randn(4, 3, generator=g, dtype=torch.float64), -1.3)]
    y = O.lora_linear(x, W, b, ads)
    for m in range(3):
        for n in range(4):
            acc = b[n].item() + sum(W[n, k].item() * x[m, k].item() for k in range(5))
            for A, B, s in ads:
                for r in range(A.shape[0]):
                    t = sum(A[r, k].item() * x[m, k].item() for k in range(5))
                    acc += s * B[n, r].item() * t
            assert abs(y[m, n].item() - acc) < 1e-12


def test_lora_invariants():
    """scale 0 == base, merged weight == unmerged, adapter order does not matter, weighted mix is linear
    (the invariants of diffusers-hf/tests/lora/utils.py:249-255, 654-698, 1066-1139)."""
    g = torch.Generator().manual_seed(1)
    x = torch.randn(7, 16, generator=g, dtype=torch.float64); W = torch.randn(12, 16, generator=g, dtype=torch.float64)
    A1, B1 = torch.randn(4, 16, generator=g, dtype=torch.float64), torch.randn(12, 4, generator=g, dtype=torch.float64)
    A2, B2 = torch.randn(2, 16, generator=g, dtype=torch.float64), torch.randn(12, 2, generator=g, dtype=torch.float64)
    base = O.lora_linear(x, W)
    assert torch.equal(O.lora_linear(x, W, None, [(A1, B1, 0.0)]), base)
    both = O.lora_linear(x, W, None, [(A1, B1, 0.8), (A2, B2, 0.6)])
    assert torch.allclose(both, O.lora_linear(x, W, None, [(A2, B2, 0.6), (A1, B1, 0.8)]), atol=1e-12)
    assert torch.allclose(both, F.linear(x, O.lora_merged_weight(W, [(A1, B1, 0.8), (A2, B2, 0.6)])), atol=1e-12)
    d1 = O.lora_linear(x, W, None, [(A1, B1, 1.0)]) - base
    d2 = O.lora_linear(x, W, None, [(A2, B2, 1.0)]) - base
    assert torch.allclose(both - base, 0.8 * d1 + 0.6 * d2, atol=1e-12)
    assert not torch.allclose(d1, d2)


def test_attention_matches_sdpa_and_brute_force():
    g = torch.Generator().manual_seed(2)
    B, H, T, S, d = 2, 3, 9, 5, 8
    q = torch.randn(B, T, H * d, generator=g); k = torch.randn(B, S, H * d, generator=g); v = torch.randn(B, S, H * d, generator=g)
    o = O.attention(q, k, v, H)
    sp = F.scaled_dot_product_attention(q.view(B, T, H, d).transpose(1, 2), k.view(B, S, H, d).transpose(1, 2),
                                        v.view(B, S, H, d).transpose(1, 2)).transpose(1, 2).reshape(B, T, H * d)
    assert torch.allclose(o, sp, atol=1e-5)
    # brute force one (b, h, t)
    b, h, t = 1, 2, 4
    qq = q[b, t, h * d:(h + 1) * d].double()
    sc = [sum((qq[i] * k[b, s, h * d + i].double()).item() for i in range(d)) / math.sqrt(d) for s in range(S)]
    mx = max(sc); w = [math.exp(z - mx) for z in sc]; z = sum(w)
    ref = [sum(w[s] / z * v[b, s, h * d + i].item() for s in range(S)) for i in range(d)]
    assert torch.allclose(o[b, t, h * d:(h + 1) * d].double(), torch.tensor(ref, dtype=torch.float64), atol=1e-5)


def test_group_norm_and_layer_norm_match_torch():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(2, 12, 5, 7, generator=g) * 3 + 1
    w = torch.randn(12, generator=g); b = torch.randn(12, generator=g)
    assert torch.allclose(O.group_norm(x, 4, w, b, 1e-5), F.group_norm(x, 4, w, b, 1e-5), atol=1e-5)
    assert torch.allclose(O.group_norm(x, 4, w, b, 1e-6, "silu"), F.silu(F.group_norm(x, 4, w, b, 1e-6)), atol=1e-5)
    assert torch.allclose(O.group_norm(x, 3, None, None, 1e-5), F.group_norm(x, 3, None, None, 1e-5), atol=1e-5)
    y = torch.randn(4, 6, 10, generator=g)
    lw = torch.randn(10, generator=g); lb = torch.randn(10, generator=g)
    assert torch.allclose(O.layer_norm(y, lw, lb, 1e-5), F.layer_norm(y, (10,), lw, lb, 1e-5), atol=1e-5)


def test_gelu_forms_match_torch():
    x = torch.linspace(-6, 6, 241)
    assert torch.allclose(O.gelu(x), F.gelu(x), atol=1e-6)
    assert torch.allclose(O.gelu(x, "tanh"), F.gelu(x, approximate="tanh"), atol=1e-6)
    p = torch.randn(3, 8, generator=torch.Generator().manual_seed(4))
    assert torch.allclose(O.geglu(p), p[:, :4] * F.gelu(p[:, 4:]), atol=1e-6)
    assert torch.allclose(O.gelu_mul(p[:, :4], p[:, 4:]), F.gelu(p[:, :4], approximate="tanh") * p[:, 4:], atol=1e-6)


def test_residual_forms():
    g = torch.Generator().manual_seed(5)
    s = torch.randn(2, 4, 3, 3, generator=g); rs = [torch.randn(2, 4, 3, 3, generator=g) for _ in range(3)]
    assert torch.allclose(O.residual_add(s, rs), s + (rs[0] + rs[1] + rs[2]) / 3)
    assert torch.equal(O.residual_add(s, rs[:1]), s + rs[0])
    h = torch.randn(2, 5, 3, 3, generator=g)
    c = O.concat_residual(h, s, rs[:1])
    assert c.shape == (2, 9, 3, 3) and torch.equal(c[:, :5], h) and torch.equal(c[:, 5:], s + rs[0])
    assert torch.equal(O.concat_residual(h, s), torch.cat([h, s], 1))


def test_sgmv_is_per_request_lora():
    g = torch.Generator().manual_seed(6)
    x = torch.randn(10, 6, generator=g); W = torch.randn(4, 6, generator=g)
    ads = [(torch.randn(2, 6, generator=g), torch.randn(4, 2, generator=g), 0.5),
           (torch.randn(3, 6, generator=g), torch.randn(4, 3, generator=g), 2.0)]
    y = O.sgmv(x, [0, 3, 7, 10], [1, -1, 0], ads, F.linear(x, W))
    assert torch.allclose(y[0:3], O.lora_linear(x[0:3], W, None, [ads[1]]), atol=1e-6)
    assert torch.equal(y[3:7], F.linear(x[3:7], W))
    assert torch.allclose(y[7:10], O.lora_linear(x[7:10], W, None, [ads[0]]), atol=1e-6)


def test_lora_conv2d_equals_conv_with_merged_kernel():
    """LoRA on a convolution == the convolution with the fused kernel W + s * (B.flatten(1) @ A.flatten(1)).reshape(W)
    (diffusers-hf/src/diffusers/models/lora.py:409-421), for stride 1 and 2, two adapters; plus a brute-force pixel."""
    import torch
    import torch.nn.functional as F
    from oracle import ops as O

    g = torch.Generator().manual_seed(0)
    x = torch.randn(2, 6, 9, 7, generator=g, dtype=torch.float64)
    w = torch.randn(5, 6, 3, 3, generator=g, dtype=torch.float64)
    b = torch.randn(5, generator=g, dtype=torch.float64)
    ads = [(torch.randn(4, 6, 3, 3, generator=g, dtype=torch.float64), torch.randn(5, 4, 1, 1, generator=g, dtype=torch.float64), 0.7),
           (torch.randn(2, 6, 3, 3, generator=g, dtype=torch.float64), torch.randn(5, 2, generator=g, dtype=torch.float64), -1.3)]
    for stride in (1, 2):
        got = O.lora_conv2d(x, w, b, ads, stride=stride, padding=1)
        wm = w.clone()
        for A, B, s in ads:
            wm = wm + s * (B.reshape(5, -1) @ A.flatten(1)).reshape(w.shape)
        assert torch.allclose(got, F.conv2d(x, wm, b, stride=stride, padding=1), atol=1e-10)
    assert torch.equal(O.lora_conv2d(x, w, b, [(ads[0][0], ads[0][1], 0.0)]), F.conv2d(x, w, b, padding=1))
    # one output pixel by hand: n=1, co=3, (h, w) = (4, 2), stride 1
    got = O.lora_conv2d(x, w, b, ads[:1])
    acc = b[3].clone()
    for ci in range(6):
        for kh in range(3):
            for kw in range(3):
                hh, ww = 4 + kh - 1, 2 + kw - 1
                if 0 <= hh < 9 and 0 <= ww < 7:
                    eff = w[3, ci, kh, kw] + 0.7 * sum(ads[0][1][3, r, 0, 0] * ads[0][0][r, ci, kh, kw] for r in range(4))
                    acc = acc + eff * x[1, ci, hh, ww]
    assert abs(got[1, 3, 4, 2] - acc) < 1e-9
