#!/usr/bin/env python3
"""Benchmark of the adapter-augmented SDXL UNet step on one MI355X.

Workload (BASELINE.json configs[2], the configuration the metric is quoted on): one bf16
UNet2DConditionModel denoising step, random-init SDXL weights, latent [2,4,128,128] (CFG batch 2,
1024x1024), t=500, context [2,77,2048], pooled text [2,1280], time_ids [2,6]; two LoRAs (rank 64 scale
0.8, rank 32 scale 0.6) on all 722 attention / feed-forward / projection linears, one ControlNet
residual set (9 down + 1 mid, ~N(0,0.1)).  A step = one HIP-graph replay of the whole forward, inputs
resident in HBM.

Prints ONE JSON line: ms per step (value), the adapter-free step beside it, a `roofline` object for the
dominant kernel (the fused LoRA GEMM: algorithmic FLOPs of all its launches in a step, counted on the adapters'
true ranks, / the sum of their durations, each launch timed with its own HIP event pair on the launch stream),
`rooflines` for the other kernels of the path (attention and convolution against the MFMA peak; GroupNorm,
LayerNorm, residual injection and the segmented shrink / expand against the HBM peak; one summary row each, their
per-shape tables go to gpurun_out/bench_details.json) and a `cpu_baseline` object (ONE full step of the fp32 CPU oracle on
the host's cores, with the FLOP-scaled mid-block sample beside it as a cross-check).  The figures the LoRA-cost target
is stated on (adapter-free step, overhead fraction) sit inside `roofline`.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA peak used for every fraction below
PEAK_HBM_GBS = 8000.0


def lora_linear_flops(M, N, K, R):
    return 2.0 * M * K * N + 2.0 * M * R * (K + N)


def build_product(device, seed=0):
    import torch
    from katz_amd.unet_2d_condition import UNet2DConditionModel, UNetConfig

    torch.manual_seed(seed)
    with torch.device(device):
        unet = UNet2DConditionModel(UNetConfig.sdxl())
    return unet.to_runtime(device, torch.bfloat16)


LORA_SPECS = (("r64", 64, 0.8), ("r32", 32, 0.6))   # (adapter name, rank, weight): BASELINE.json configs[2]


def add_random_loras(unet, device, specs=LORA_SPECS, seed=10):
    import torch

    g = torch.Generator(device=device).manual_seed(seed)
    for name, rank, _ in specs:
        for lin in unet.lora_linears().values():
            down = (torch.randn(rank, lin.in_features, generator=g, device=device) * 0.02).to(torch.bfloat16)
            up = (torch.randn(lin.out_features, rank, generator=g, device=device) * 0.02).to(torch.bfloat16)
            lin.add_adapter(name, down, up, alpha=None)
    return [s[0] for s in specs], [s[2] for s in specs]


def make_inputs(device, seed=1):
    import torch

    g = torch.Generator(device=device).manual_seed(seed)
    bf = torch.bfloat16
    rn = lambda *s, std=1.0: (torch.randn(*s, generator=g, device=device) * std).to(bf)
    sample = rn(2, 4, 128, 128).contiguous(memory_format=torch.channels_last)
    ctx = rn(2, 77, 2048)
    added = dict(text_embeds=rn(2, 1280),
                 time_ids=torch.tensor([[1024, 1024, 0, 0, 1024, 1024]] * 2, dtype=torch.float32, device=device))
    shapes = [(320, 128)] * 3 + [(320, 64), (640, 64), (640, 64), (640, 32), (1280, 32), (1280, 32)]
    down = [rn(2, c, h, h, std=0.1).contiguous(memory_format=torch.channels_last) for c, h in shapes]
    mid = rn(2, 1280, 32, 32, std=0.1).contiguous(memory_format=torch.channels_last)
    t = torch.tensor([500.0], device=device)
    return sample, t, ctx, added, down, mid


def time_graph(step, steps, warmup):
    import torch

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def instrumented_step(unet, inputs):
    """One eager step with per-launch HIP events on every katz_hip kernel.  The stream is first plugged
    with a spin kernel so that all launches are queued behind it and then run back to back, as they do
    in the graph."""
    import torch
    from katz_amd import ops

    sample, t, ctx, added, down, mid = inputs
    conv_flops = [0.0]

    def hook(m, inp, out):
        kh, kw = m.kernel_size
        conv_flops[0] += 2.0 * out.numel() * m.in_channels * kh * kw

    hooks = [m.register_forward_hook(hook) for m in unet.modules() if isinstance(m, torch.nn.Conv2d)]
    ops.CALL_LOG = []
    torch.cuda.synchronize()
    torch.cuda._sleep(int(0.08 * 2.4e9))
    ops.profile_begin()
    try:
        with torch.no_grad():
            unet(sample, t, ctx, added_cond_kwargs=added, down_block_additional_residuals=down,
                 mid_block_additional_residual=mid)
    finally:
        launches = ops.profile_end()
        log, ops.CALL_LOG = ops.CALL_LOG, None
        for h in hooks:
            h.remove()
    torch.cuda.synchronize()
    return launches, log, conv_flops[0]


def host_cores():
    """Threads for the CPU baseline: the share of the host this job has been given (OMP_NUM_THREADS, which the GPU
    boxes set to their per-GPU share of cores), never more than the CPUs visible."""
    n = os.cpu_count() or 1
    try:
        n = min(n, int(os.environ.get("OMP_NUM_THREADS", n)))
    except ValueError:
        pass
    return max(n, 1)


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def sgmv_rooflines(dev):
    """Segmented shrink / expand (BASELINE.json configs[3]: 8 requests, one adapter each, ranks from {8..128}) at the
    two SDXL widths, timed per launch with HIP events; algorithmic bytes: shrink 2(sum T K + sum r K + sum T r), expand
    2(sum T r + sum r N + 2 sum T N) (y is read, updated and written)."""
    import torch
    from katz_amd import ops

    bf = torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(2)
    rn = lambda *s, std=1.0: (torch.randn(*s, device=dev, generator=g) * std).to(bf)
    ranks = [64, 8, 128, 32, 16, 64, 128, 32]
    rows = {"shrink": [], "expand": [], "fused": []}
    for T, K, N in ((4096, 640, 640), (1024, 1280, 1280), (77, 2048, 1280)):
        RP = 128
        # several input sets, used in turn, together larger than the 256 MB memory-side cache: a launch does not find
        # its operands left there by the previous launch on the same buffers
        nbuf = max(2, min(12, int(400e6 // (2.0 * 8 * T * (K + 2 * N))) + 1))
        xs = [rn(8 * T, K) for _ in range(nbuf)]
        ys = [rn(8 * T, N) for _ in range(nbuf)]
        tbs = [torch.zeros(8 * T, RP, device=dev, dtype=bf) for _ in range(nbuf)]
        a_all = torch.zeros(8, RP, K, device=dev, dtype=bf)
        b_all = torch.zeros(8, N, RP, device=dev, dtype=bf)
        for i, r in enumerate(ranks):
            a_all[i, :r] = rn(r, K, std=0.02)
            b_all[i, :, :r] = rn(N, r, std=0.02)
        ss = torch.arange(0, 9 * T, T, dtype=torch.int32, device=dev)
        sa = torch.arange(8, dtype=torch.int32, device=dev)
        rp = torch.tensor([(r + 31) // 32 * 32 for r in ranks], dtype=torch.int32, device=dev)
        sc = torch.full((8,), 0.7, device=dev)
        sr = float(sum(ranks))

        def one(i):
            j = i % nbuf
            ops.sgmv_shrink(xs[j], a_all, ss, sa, rp, T, out=tbs[j])
            ops.sgmv_expand_(ys[j], tbs[j], b_all, ss, sa, rp, sc, T)
        for i in range(nbuf):
            one(i)
        torch.cuda.synchronize()
        reps = 2 * nbuf
        ops.profile_begin()
        for i in range(reps):
            one(i)
        ls = ops.profile_end()
        assert len(ls) == 2 * reps, len(ls)    # one launch per call
        # the same in one launch (t stays in the workgroup): x read, y read and written, the adapter matrices
        ops.profile_begin()
        for i in range(reps):
            j = i % nbuf
            ops.sgmv_fused_(ys[j], xs[j], a_all, b_all, ss, sa, rp, sc, T)
        lf = ops.profile_end()
        assert len(lf) == reps, len(lf)
        for kind, nbytes in (("shrink", 2.0 * (8 * T * K + sr * K + T * sr)), ("expand", 2.0 * (T * sr + sr * N + 2 * 8 * T * N)),
                             ("fused", 2.0 * (8 * T * K + sr * K + sr * N + 2 * 8 * T * N))):
            if kind == "fused":
                ds = sorted(d for _, d in lf)
            else:
                ds = sorted(d for i, (_, d) in enumerate(ls) if (i % 2 == 0) == (kind == "shrink"))   # launches alternate
            med = ds[len(ds) // 2]
            rows[kind].append({"shape": f"8 requests x {T} rows, K{K} N{N}, ranks {ranks}", "avg_us": round(med * 1e3, 2),
                               "achieved": round(nbytes / (med * 1e-3) / 1e9, 1),
                               "frac": round(nbytes / (med * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)})
    # the 77-row class (cross-attention to_k / to_v read the text context) as ONE launch over all layers of a width: 120
    # layers at 1280 (60 blocks x to_k, to_v), x shared, per-layer A / B / y from a pointer table
    T, K, N, L = 77, 2048, 1280, 120
    x = rn(8 * T, K)
    a_alls = [torch.zeros(8, 128, K, device=dev, dtype=bf) for _ in range(L)]
    b_alls = [torch.zeros(8, N, 128, device=dev, dtype=bf) for _ in range(L)]
    for a, b in zip(a_alls, b_alls):
        for i, r in enumerate(ranks):
            a[i, :r].normal_(0, 0.02, generator=g)
            b[i, :, :r].normal_(0, 0.02, generator=g)
    ys = [rn(8 * T, N) for _ in range(L)]
    ss = torch.arange(0, 9 * T, T, dtype=torch.int32, device=dev)
    table = ops.sgmv_fused_grouped_table(ys, a_alls, b_alls)
    for _ in range(2):
        ops.sgmv_fused_grouped_(ys, x, a_alls, b_alls, ss, sa, rp, sc, T, table=table)
    torch.cuda.synchronize()
    ops.profile_begin()
    for _ in range(5):
        ops.sgmv_fused_grouped_(ys, x, a_alls, b_alls, ss, sa, rp, sc, T, table=table)
    lg = sorted(d for _, d in ops.profile_end())
    assert len(lg) == 5, len(lg)
    sr = float(sum(ranks))
    nbytes = 2.0 * (8 * T * K + L * (sr * (K + N) + 2 * 8 * T * N))
    med = lg[len(lg) // 2]
    rows["fused"].append({"shape": f"8 requests x {T} rows, K{K} N{N}, {L} layers in one launch (grouped), ranks {ranks}",
                          "avg_us": round(med * 1e3, 2), "achieved": round(nbytes / (med * 1e-3) / 1e9, 1),
                          "frac": round(nbytes / (med * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)})
    del a_alls, b_alls, ys
    out = []
    for kind in ("shrink", "expand", "fused"):
        best = rows[kind][0]
        what = "shrink + expand in one launch" if kind == "fused" else kind
        out.append({"kernel": f"segmented multi-adapter {what} (kh_sgmv_{kind}_bf16), median over launches that rotate through input sets larger than the memory-side cache",
                    "bound": "hbm", "achieved": best["achieved"], "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": best["frac"],
                    "by_shape": rows[kind]})
    return out


def cpu_baseline_sample(cores, reps=3):
    """Cross-check of the full-step baseline below: the fp32 CPU oracle's UNet mid block (resnet, 10 transformer blocks
    with both LoRAs, resnet; batch 2, 32x32 latent), to be scaled to a whole step by algorithmic FLOPs."""
    import torch
    from oracle import blocks as OB

    torch.set_num_threads(cores)
    torch.manual_seed(0)
    blk = OB.UNetMidBlock2DCrossAttn(in_channels=1280, temb_channels=1280, transformer_layers_per_block=10,
                                     resnet_eps=1e-5, num_attention_heads=20, cross_attention_dim=2048,
                                     use_linear_projection=True).eval()
    flops = 0.0
    M = 2 * 1024
    g = torch.Generator().manual_seed(10)
    for name, m in blk.named_modules():
        if isinstance(m, OB.OracleLoRALinear):
            rows = 2 * 77 if (".attn2.to_k" in name or ".attn2.to_v" in name) else M
            for an, r, w in (("r64", 64, 0.8), ("r32", 32, 0.6)):
                m.add_adapter(an, torch.randn(r, m.in_features, generator=g) * 0.02,
                              torch.randn(m.out_features, r, generator=g) * 0.02, None, w)
            m.active = ["r64", "r32"]
            flops += lora_linear_flops(rows, m.out_features, m.in_features, 96)
        elif isinstance(m, torch.nn.Conv2d):
            flops += 2.0 * 2 * 1024 * m.out_channels * m.in_channels * m.kernel_size[0] * m.kernel_size[1]
    flops += 10 * (4.0 * 2 * 20 * 1024 * 1024 * 64 + 4.0 * 2 * 20 * 1024 * 77 * 64)
    x = torch.randn(2, 1280, 32, 32, generator=g)
    temb = torch.randn(2, 1280, generator=g)
    ctx = torch.randn(2, 77, 2048, generator=g)
    with torch.no_grad():
        blk(x, temb, ctx)  # warm-up
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            blk(x, temb, ctx)
            ts.append(time.perf_counter() - t0)
    ts.sort()
    return ts[len(ts) // 2], flops


def cpu_baseline_full_step(cores):
    """ONE full step of BASELINE.json configs[2] on the fp32 CPU oracle (oracle/unet_sdxl.py, the restatement of the
    reference's diffusers path: 2.57 B parameters, both LoRAs unmerged on all 722 linears, the 9 + 1 ControlNet residuals),
    on `cores` threads.  The weights are random (their values do not change the time): the model is created without
    torch's initialisers and filled from one pool of normal numbers scaled per tensor, which takes seconds instead of
    a minute.  Returns the seconds of the one timed step."""
    import torch
    from oracle.unet_sdxl import UNet2DConditionModel as OracleUNet, UNetConfig as OracleCfg

    torch.set_num_threads(cores)
    with torch.device("meta"):
        model = OracleUNet(OracleCfg.sdxl())
    model = model.to_empty(device="cpu").eval()
    g = torch.Generator().manual_seed(0)
    pool = torch.randn(1 << 24, generator=g)

    def fill(t, std):
        flat = t.view(-1)
        for o in range(0, flat.numel(), pool.numel()):
            n = min(pool.numel(), flat.numel() - o)
            torch.mul(pool[:n], std, out=flat[o:o + n])

    with torch.no_grad():
        for name, p in model.named_parameters():
            if p.dim() > 1:
                fill(p.data, (3.0 * p[0].numel()) ** -0.5)      # the spread of torch's default Linear / Conv2d init
            elif name.endswith("weight"):
                p.fill_(1.0)                                     # norm scales
            else:
                p.zero_()
        for k, m in enumerate(model.lora_linears().values()):
            for an, r, w in (("r64", 64, 0.8), ("r32", 32, 0.6)):
                o = (k * 7919 * 64) % (pool.numel() - r * (m.in_features + m.out_features))
                down = (pool[o:o + r * m.in_features] * 0.02).view(r, m.in_features)
                up = (pool[o + r * m.in_features:o + r * (m.in_features + m.out_features)] * 0.02).view(m.out_features, r)
                m.add_adapter(an, down, up, None, w)
        model.set_adapters(["r64", "r32"], [0.8, 0.6])
        rn = lambda *s, std=1.0: torch.randn(*s, generator=g) * std
        x, ctx = rn(2, 4, 128, 128), rn(2, 77, 2048)
        added = dict(text_embeds=rn(2, 1280), time_ids=torch.tensor([[1024.0, 1024, 0, 0, 1024, 1024]] * 2))
        shapes = [(320, 128)] * 3 + [(320, 64), (640, 64), (640, 64), (640, 32), (1280, 32), (1280, 32)]
        down = [rn(2, c, h, h, std=0.1) for c, h in shapes]
        mid = rn(2, 1280, 32, 32, std=0.1)
        t0 = time.perf_counter()
        out = model(x, 500, ctx, added, down, mid)
        sec = time.perf_counter() - t0
    if out.shape != (2, 4, 128, 128) or not bool(torch.isfinite(out).all()):
        raise RuntimeError("cpu_baseline: the oracle step did not produce a finite [2,4,128,128] output")
    return sec


PROFILE_SUMMARY = ROOT / "profiles" / "kernels_at_baseline_shapes_mfma_busy_and_hbm_traffic.txt"


def traffic_from_profiles(kernel_prefix):
    """HBM-side bytes per launch (read + written) of the first row of the committed counter summary whose name starts
    with `kernel_prefix`, with the row it came from; (None, reason) when the summary or the row is missing.  The
    summary is written from two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE) of `bench.py --kernel-probe`, each
    calibrated against a copy of known size; it is a record of that run, not a measurement of this one."""
    import re

    if not PROFILE_SUMMARY.exists():
        return None, f"{PROFILE_SUMMARY.name} not found"
    for line in PROFILE_SUMMARY.read_text().splitlines():
        if line.startswith(kernel_prefix):
            m = re.search(r"hbm rd\s+([0-9.]+)\s+wr\s+([0-9.]+)\s+MB", line)
            if m:
                return (float(m.group(1)) + float(m.group(2))) * 1e6, " ".join(line.split())
    return None, f"no row {kernel_prefix!r} in {PROFILE_SUMMARY.name}"


def kernel_probe():
    """Counter / trace run of the individual kernels at the shapes of BASELINE.json's configurations, three times
    each, preceded by a 64 MiB device copy of known size (the calibration of FETCH_SIZE / WRITE_SIZE).
    Used as  rocprofv3 --kernel-trace --stats -- python3 bench.py --kernel-probe  (durations) and
    rocprofv3 --pmc <counter> -- python3 bench.py --kernel-probe  (one counter per run).  Prints, as JSON, the
    algorithmic FLOPs / bytes of every probed launch in launch order."""
    import torch
    from katz_amd import ops

    dev = torch.device("cuda:0")
    bf = torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s, std=1.0: (torch.randn(*s, device=dev, generator=g) * std).to(bf)
    cl = lambda t: t.contiguous(memory_format=torch.channels_last)
    src = torch.randn(16 << 20, device=dev, generator=g)            # 64 MiB fp32
    dst = torch.empty_like(src)
    runs, meta = [], []

    def add(name, fn, flops=0.0, nbytes=0.0):
        runs.append(fn)
        meta.append({"kernel": name, "algorithmic_flops": flops, "algorithmic_bytes": nbytes})

    # K1: largest LoRA linear (GEGLU projection) and the most frequent one (d x d), as shrink + GEMM
    for (M, K, N, geglu) in ((2048, 1280, 10240, True), (2048, 1280, 1280, False), (8192, 640, 640, False)):
        R = 128
        x, w, b = rn(M, K), rn(N, K, std=0.02), rn(N)
        a_cat, b_cat = rn(R, K, std=0.02), rn(N, R, std=0.02)
        scale = torch.full((R,), 0.8, device=dev)
        tbuf = torch.empty(M, R, device=dev, dtype=bf)
        nout = N // 2 if geglu else N
        add(f"lora_shrink M{M} K{K} R{R}", lambda x=x, a=a_cat, s=scale, t=tbuf: ops.lora_shrink(x, a, s, out=t),
            2.0 * M * K * R, 2.0 * (M * K + R * K + M * R))
        add(f"lora_gemm M{M} K{K} N{N} R{R}{' geglu' if geglu else ''}",
            lambda x=x, w=w, b=b, t=tbuf, bc=b_cat, ge=geglu: ops.lora_linear_pre(x, w, b, t, bc, geglu=ge),
            2.0 * M * N * (K + R), 2.0 * (M * K + K * N + M * nout + R * N + M * R))
    # the d x d layer again as ONE launch: the shrink on the CUs its 160 GEMM tiles leave idle
    M, K, N, R = 2048, 1280, 1280, 128
    x, w, b = rn(M, K), rn(N, K, std=0.02), rn(N)
    a_cat, b_cat = rn(R, K, std=0.02), rn(N, R, std=0.02)
    scale = torch.full((R,), 0.8, device=dev)
    add(f"lora_linear_split M{M} K{K} N{N} R{R} (shrink in launch)",
        lambda x=x, w=w, b=b, a=a_cat, s=scale, bc=b_cat: ops.lora_linear_split(x, w, b, a, s, bc),
        2.0 * M * N * (K + R) + 2.0 * M * K * R, 2.0 * (M * K + K * N + M * N + R * N + R * K))
    # ... and as the step runs it: ranks 64 + 32 in 128 packed columns (r_used = 96), the in-launch shrink on 64 x 32 tiles
    Rt = 96
    a96, b96 = a_cat.clone(), b_cat.clone()
    a96[Rt:] = 0
    b96[:, Rt:] = 0
    add(f"lora_linear_split M{M} K{K} N{N} R{R} r_used {Rt} (shrink in launch, 64x32 tiles)",
        lambda x=x, w=w, b=b, a=a96, s=scale, bc=b96: ops.lora_linear_split(x, w, b, a, s, bc, r_used=96),
        2.0 * M * N * (K + Rt) + 2.0 * M * K * Rt, 2.0 * (M * K + K * N + M * N + Rt * N + Rt * K))
    # the N 640 layer of the 64 x 64 level as ONE launch: every workgroup of the 128 x 160 tiles computes a piece of T first
    M, K, N = 8192, 640, 640
    x8, w8, b8 = rn(M, K), rn(N, K, std=0.02), rn(N)
    a8, bc8 = rn(R, K, std=0.02), rn(N, R, std=0.02)
    a8[Rt:] = 0
    bc8[:, Rt:] = 0
    add(f"lora_linear_split M{M} K{K} N{N} R{R} r_used {Rt} (cooperative shrink in launch)",
        lambda: ops.lora_linear_split(x8, w8, b8, a8, scale, bc8, r_used=96),
        2.0 * M * N * (K + Rt) + 2.0 * M * K * Rt, 2.0 * (M * K + K * N + M * N + Rt * N + Rt * K))
    # K3: attention at the three SDXL shapes
    for (B, H, T, S) in ((2, 10, 4096, 4096), (2, 20, 1024, 1024), (2, 20, 1024, 77)):
        q, k, v = rn(B, T, H * 64), rn(B, S, H * 64), rn(B, S, H * 64)
        add(f"attention B{B} H{H} T{T} S{S}", lambda q=q, k=k, v=v, H=H: ops.attention(q, k, v, H),
            4.0 * B * H * T * S * 64, 2.0 * 64 * B * H * (2 * T + 2 * S))
    # K3b: the text cross-attention of the 32x32 level inside its query projection's launch (adapters: shrink in launch)
    B, H, T, S, K, R = 2, 20, 1024, 77, 1280, 128
    xq, wq, kx, vx = rn(B, T, K), rn(H * 64, K, std=0.02), rn(B, S, H * 64), rn(B, S, H * 64)
    aq, bq, sq = rn(R, K, std=0.02), rn(H * 64, R, std=0.02), torch.full((R,), 0.8, device=dev)
    add(f"lora_linear_xattn M{B * T} K{K} N{H * 64} R{R} S{S} (to_q + attention)",
        lambda: ops.lora_linear_xattn(xq, wq, kx, vx, H, a_cat=aq, col_scale=sq, b_cat=bq),
        2.0 * B * T * H * 64 * (K + R) + 2.0 * B * T * K * R + 4.0 * B * H * T * S * 64,
        2.0 * (B * T * K + K * H * 64 + B * T * H * 64 + R * H * 64 + R * K + 2 * B * S * H * 64))
    # K2: segmented shrink / expand, 8 requests x 4096 tokens, d = 640, one adapter each (ranks 8 .. 128)
    T, dm, RP = 4096, 640, 128
    ranks = [64, 8, 128, 32, 16, 64, 128, 32]
    x = rn(8 * T, dm)
    a_all, b_all = torch.zeros(8, RP, dm, device=dev, dtype=bf), torch.zeros(8, dm, RP, device=dev, dtype=bf)
    for i, r in enumerate(ranks):
        a_all[i, :r] = rn(r, dm, std=0.02)
        b_all[i, :, :r] = rn(dm, r, std=0.02)
    ss = torch.arange(0, 9 * T, T, dtype=torch.int32, device=dev)
    sa = torch.arange(8, dtype=torch.int32, device=dev)
    rp = torch.tensor([(r + 31) // 32 * 32 for r in ranks], dtype=torch.int32, device=dev)
    sc = torch.full((8,), 0.7, device=dev)
    y = rn(8 * T, dm)
    tb = torch.zeros(8 * T, RP, device=dev, dtype=bf)
    sr = float(sum(ranks))
    add("sgmv_shrink 8x4096x640", lambda: ops.sgmv_shrink(x, a_all, ss, sa, rp, T, out=tb), 2.0 * T * dm * sr,
        2.0 * (8 * T * dm + sr * dm + T * sr))
    add("sgmv_expand 8x4096x640", lambda: ops.sgmv_expand_(y, tb, b_all, ss, sa, rp, sc, T), 2.0 * T * dm * sr,
        2.0 * (T * sr + sr * dm + 2 * 8 * T * dm))
    y2 = rn(8 * T, dm)
    add("sgmv_fused 8x4096x640", lambda: ops.sgmv_fused_(y2, x, a_all, b_all, ss, sa, rp, sc, T), 4.0 * T * dm * sr,
        2.0 * (8 * T * dm + sr * dm + sr * dm + 2 * 8 * T * dm))
    # K4 / K5: norms and the ControlNet residual injection
    xg, gam, bet = cl(rn(2, 320, 128, 128)), rn(320), rn(320)
    add("group_norm+silu 2x320x128x128 nhwc", lambda: ops.group_norm(xg, 32, gam, bet, 1e-5, "silu"), 0.0, 4.0 * xg.numel())
    xl, gl, bl = rn(2048, 1280), rn(1280), rn(1280)
    add("layer_norm 2048x1280", lambda: ops.layer_norm(xl, gl, bl), 0.0, 4.0 * xl.numel())
    h, skip, res = cl(rn(2, 320, 128, 128)), cl(rn(2, 320, 128, 128)), cl(rn(2, 320, 128, 128, std=0.1))
    add("concat_residual 2x(320+320)x128x128", lambda: ops.concat_residual(h, skip, [res]), 0.0, 2.0 * (3 + 2) * h.numel())
    mid, rmid = cl(rn(2, 1280, 32, 32)), cl(rn(2, 1280, 32, 32, std=0.1))
    add("residual_add 2x1280x32x32", lambda: ops.residual_add_(mid, [rmid]), 0.0, 2.0 * 3 * mid.numel())
    # K1c: a 3x3 convolution of the 64x64 level
    xc, wc, bc = cl(rn(2, 640, 64, 64)), ops.pack_conv3x3_weight(rn(640, 640, 3, 3, std=0.01)), rn(640)
    add("conv3x3 640->640 @64x64", lambda: ops.conv3x3(xc, wc, bc), 2.0 * 8192 * 640 * 5760,
        2.0 * (xc.numel() + wc.numel() + 8192 * 640))
    # the tail of a denoising step: conv_out with guidance + Euler in its epilogue
    xo, wo, bo = cl(rn(2, 320, 128, 128)), ops.pack_conv3x3_weight(rn(4, 320, 3, 3, std=0.02)), rn(4)
    lat = cl(rn(1, 4, 128, 128))
    nxt = cl(torch.empty(2, 4, 128, 128, device=dev, dtype=bf))
    coef = torch.tensor([4.2, 3.1, (3.1 ** 2 + 1) ** 0.5], device=dev)
    add("conv_out + guidance + Euler 2x320x128x128", lambda: ops.conv_out_cfg_euler(xo, wo, bo, lat, coef, 7.5, model_input_next=nxt),
        2.0 * 32768 * 2880 * 4, 2.0 * (xo.numel() + wo.numel() + 2 * lat.numel() + nxt.numel()))
    torch.cuda.synchronize()
    for _ in range(3):
        dst.copy_(src)
        for fn in runs:
            fn()
    torch.cuda.synchronize()
    print(json.dumps({"kernel_probe": {"copy_bytes_read": src.numel() * 4, "copy_bytes_written": src.numel() * 4,
                                       "launches_per_round": meta, "rounds": 3}}))


def merge_probe():
    """Katz's per-request merge (patch_on_lora, pipeline_controlnet_sd_xl_katz.py:1730-1770: 0.090 / 0.123 s on H800
    in the reference's logs) on the SDXL UNet: a rank-64 adapter on all 722 linears merged by the batched merge kernel.
    Timed three ways: adapters in pageable host memory as float16 (what the shared-memory segments are; the upload is
    part of the time, as in the reference), adapters already resident on the GPU, and the merge launch alone (HIP
    events).  Prints one JSON line."""
    import torch
    from katz_amd import ops
    from katz_amd.shm_adapters import KATZ_MERGE_SCALE, patch_on_lora

    dev = torch.device("cuda:0")
    unet = build_product(dev)
    lin = unet.lora_linears()
    g = torch.Generator().manual_seed(4)
    host_sd, key_match = {}, {}
    for name, m in lin.items():
        host_sd[name + ".down"] = (torch.randn(64, m.in_features, generator=g) * 1e-3).to(torch.float16)
        host_sd[name + ".up"] = (torch.randn(m.out_features, 64, generator=g) * 1e-3).to(torch.float16)
        key_match[name + ".weight"] = {"lora_down_key": name + ".down", "lora_up_key": name + ".up"}
    dev_sd = {k: v.to(dev) for k, v in host_sd.items()}
    n_bytes = sum(v.numel() * 2 for v in host_sd.values())
    w_bytes = sum(m.weight.numel() * 2 for m in lin.values())

    def timed(sd, sign):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        n = patch_on_lora(unet, sd, key_match, scale=sign * KATZ_MERGE_SCALE)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3, n

    timed(dev_sd, 1.0); timed(dev_sd, -1.0)   # warm-up
    host_ms = [timed(host_sd, s)[0] for s in (1.0, -1.0, 1.0, -1.0)]
    dev_ms = [timed(dev_sd, s)[0] for s in (1.0, -1.0, 1.0, -1.0)]
    ops.profile_begin()
    timed(dev_sd, 1.0); timed(dev_sd, -1.0)
    kernel_ms = [d for n, d in ops.profile_end() if n == "lora_merge"]
    finite = all(bool(torch.isfinite(m.weight).all()) for m in list(lin.values())[:20])
    print(json.dumps({
        "metric": "patch_on_lora_ms_sdxl_722_linears_rank64", "unit": "ms",
        "value_adapters_in_pageable_host_memory": round(min(host_ms), 2),
        "value_adapters_resident_on_gpu": round(min(dev_ms), 2),
        "merge_kernel_ms": round(min(kernel_ms), 3), "layers": len(lin),
        "adapter_bytes": n_bytes, "weight_bytes_read_plus_written": 2 * w_bytes,
        "merge_kernel_GBps": round((2 * w_bytes + n_bytes) / (min(kernel_ms) * 1e-3) / 1e9, 1),
        "reference_h800_s": [0.090, 0.123], "all_runs_ms": {"host": [round(x, 2) for x in host_ms], "gpu": [round(x, 2) for x in dev_ms]},
        "weights_finite": finite}))


def loop_bench(args):
    """BASELINE.json configs[4]: the 50-step guided denoise loop at 1024x1024 -- random-init SDXL UNet with the two
    LoRAs, random-init SDXL-size ControlNet (from_unet, conditioning image [2,3,1024,1024] uniform[0,1], scale 0.5),
    Euler discrete scheduler (SDXL schedule), guidance 7.5, seeded latents x init_noise_sigma; every step is one replay
    of one captured graph holding ControlNet -> UNet -> guidance + Euler.  Prints one JSON line: end-to-end ms of the
    loop, ms per step, and the per-kernel breakdown of one step (per-launch HIP events on an eager step)."""
    import torch
    from katz_amd import ops
    from katz_amd.controlnet import ControlNetModel
    from katz_amd.graph import GraphedDenoiseStep
    from katz_amd.scheduler import EulerDiscreteScheduler

    dev = torch.device("cuda:0")
    bf = torch.bfloat16
    torch.manual_seed(0)
    with torch.device(dev):
        from katz_amd.unet_2d_condition import UNet2DConditionModel, UNetConfig
        unet = UNet2DConditionModel(UNetConfig.sdxl())
        cn = ControlNetModel.from_unet(unet)
        g = torch.Generator(device=dev).manual_seed(3)
        with torch.no_grad():   # a trained ControlNet's "zero" convolutions are not zero: small random ones
            for m in [cn.controlnet_cond_embedding.conv_out, cn.controlnet_mid_block, *cn.controlnet_down_blocks]:
                m.weight.copy_(torch.randn(m.weight.shape, generator=g, device=dev) * (0.1 / m.weight[0].numel() ** 0.5))
    unet, cn = unet.to_runtime(dev, bf), cn.to_runtime(dev, bf)
    names, weights = add_random_loras(unet, dev)
    unet.set_adapters(names, weights)
    sample, t, ctx, added, _, _ = make_inputs(dev)
    cond = torch.rand(2, 3, 1024, 1024, generator=g, device=dev).to(bf)
    sch = EulerDiscreteScheduler(beta_start=0.00085, beta_end=0.012, beta_schedule="scaled_linear",
                                 timestep_spacing="leading", steps_offset=1)
    sch.set_timesteps(args.loop_steps, device=dev)
    lat0 = (torch.randn(1, 4, 128, 128, generator=g, device=dev) * sch.init_noise_sigma).to(bf)
    with torch.no_grad():
        step = GraphedDenoiseStep(unet, cn, lat0, ctx, added, cond, 7.5, 0.5, hoist_context_kv=not args.context_kv_per_step)
        for _ in range(args.warmup_loops):
            out = step.run(lat0, sch)
        torch.cuda.synchronize()
        times = []
        for _ in range(args.loops):
            t0 = time.perf_counter()
            out = step.run(lat0, sch, check=False)
            torch.cuda.synchronize()
            times.append((time.perf_counter() - t0) * 1e3)
        ops.check_split_timeouts(dev)
        finite = bool(torch.isfinite(out.float()).all())
        # the same loop with the UNet alone (zero-cost ControlNet): what the ControlNet adds per step
        # per-kernel breakdown of one eager step
        model_input = torch.cat([lat0] * 2).contiguous(memory_format=torch.channels_last)
        emb = cn.embed_condition(cond)
        torch.cuda.synchronize()
        torch.cuda._sleep(int(0.1 * 2.4e9))
        ops.profile_begin()
        try:
            d, m = cn(model_input, t, ctx, cond, 0.5, added_cond_kwargs=added, cond_embedding=emb)
            n_cn = None
            eps = unet(model_input, t, ctx, added_cond_kwargs=added, down_block_additional_residuals=d,
                       mid_block_additional_residual=m).sample
            ops.cfg_euler_step(eps, lat0.contiguous(memory_format=torch.channels_last), sch.coef_table(dev)[0], 7.5)
        finally:
            launches = ops.profile_end()
        torch.cuda.synchronize()
        torch.cuda._sleep(int(0.1 * 2.4e9))
        ops.profile_begin()
        try:
            cn.embed_condition(cond)
        finally:
            emb_launches = ops.profile_end()
    by_kernel = {}
    for name, dur in launches:
        e = by_kernel.setdefault(name, [0, 0.0])
        e[0] += 1
        e[1] += dur
    times.sort()
    med = times[len(times) // 2]
    result = {
        "metric": "denoise_loop_ms_1024_2lora_1cn", "value": round(med, 2), "unit": "ms", "n_gpus": 1,
        "loops_timed": args.loops, "loop_steps": args.loop_steps, "ms_per_step": round(med / args.loop_steps, 3),
        "higher_is_better": False, "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic (random-init SDXL UNet and ControlNet, seeded latents, conditioning image uniform[0,1])",
        "config": {"workload": f"{args.loop_steps}-step SDXL denoise loop at 1024x1024: per step ControlNet (SDXL arch, image "
                               "[2,3,1024,1024], scale 0.5) -> UNet (2 LoRAs r64 s0.8 + r32 s0.6, CFG batch 2) -> guidance 7.5 + "
                               "Euler discrete; one HIP graph replay per step" + ("; inside the graph the ControlNet runs on a second stream "
                               "beside the UNet's down and mid blocks" if step.overlap else "") +
                               "; conditioning embedding" + (" and the text context's K / V projections" if step.hoist_kv else "") +
                               " computed once per loop",
                   "global_batch": 2, "parallelism": "single GPU"},
        "roofline": {"kernel": "whole loop (every kernel of ControlNet + UNet + scheduler step); per-kernel rooflines are in the default mode's line",
                     "loop_ms": round(med, 2), "ms_per_step": round(med / args.loop_steps, 3), "loop_steps": args.loop_steps},
        "loop_ms_all": [round(x, 2) for x in times], "output_finite": finite,
        "kernel_ms_per_step": {k: {"launches": v[0], "ms": round(v[1], 3)} for k, v in sorted(by_kernel.items())},
        "kernel_ms_sum_per_step": round(sum(v[1] for v in by_kernel.values()), 3),
        "controlnet_beside_unet": bool(step.overlap),
        "cond_embedding_once_per_loop_ms": round(sum(d for _, d in emb_launches), 3),
    }
    print(json.dumps(result))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--loop", action="store_true",
                    help="BASELINE configs[4]: the 50-step ControlNet + UNet + Euler denoise loop, end-to-end ms")
    ap.add_argument("--merge-probe", action="store_true",
                    help="time Katz's patch_on_lora (merge of a rank-64 adapter into all 722 SDXL linears)")
    ap.add_argument("--loop-steps", type=int, default=50)
    ap.add_argument("--loops", type=int, default=3)
    ap.add_argument("--warmup-loops", type=int, default=1)
    ap.add_argument("--context-kv-per-step", action="store_true",
                    help="--loop: project the text context's K / V inside every step (as the reference does) instead of once per loop")
    ap.add_argument("--kernel-probe", action="store_true",
                    help="run only a 64 MiB copy and each kernel at its BASELINE shapes three times (for rocprofv3)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU only (no collectives, no sharding); --gpus must be 1",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from katz_amd.graph import GraphedUNetStep

    if args.kernel_probe:
        kernel_probe()
        return
    if args.merge_probe:
        merge_probe()
        return
    if args.loop:
        if not torch.cuda.is_available():
            print("bench.py: no GPU visible; the katz_hip kernels have no CPU path", file=sys.stderr)
            sys.exit(1)
        loop_bench(args)
        return

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the katz_hip kernels have no CPU path", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    unet = build_product(dev)
    names, weights = add_random_loras(unet, dev)
    inputs = make_inputs(dev)
    sample, t, ctx, added, down, mid = inputs

    with torch.no_grad():
        # adapter-free step (same ControlNet residuals) for the LoRA-cost comparison
        unet.set_adapters([], [])
        g0 = GraphedUNetStep(unet, sample, t, ctx, added, down, mid)
        ms_free = time_graph(g0, args.steps, args.warmup)
        del g0
        unet.set_adapters(names, weights)
        g1 = GraphedUNetStep(unet, sample, t, ctx, added, down, mid)
        ms = time_graph(g1, args.steps, args.warmup)
        out = g1().float()
        finite = bool(torch.isfinite(out).all())
        del g1
        launches, log, conv_flops = instrumented_step(unet, inputs)

    from katz_amd import ops

    ops.check_split_timeouts(dev)   # a bounded in-launch wait that ran out would make every number below meaningless

    # ---- per-kernel accounting of the instrumented step --------------------------------------------------------
    true_rank = sum(r for _, r, _ in LORA_SPECS)       # 64 + 32: FLOPs are counted on the adapters' ranks, not on the
    by_kernel = {}                                     # 128 columns they are padded to (the kernels skip the padding)
    for name, dur in launches:
        e = by_kernel.setdefault(name, [0, 0.0])
        e[0] += 1
        e[1] += dur
    # (a cross-attention's query projection that runs the attention in its epilogue is one launch of the GEMM family)
    gemm_calls = [c for c in log if c[0] in ("lora_linear", "lora_linear_grouped", "lora_linear_xattn")]
    gemm_ms = [d for n, d in launches if n == "lora_gemm"]
    assert len(gemm_calls) == len(gemm_ms), (len(gemm_calls), len(gemm_ms))
    # two-launch layers: the shrink launch belongs to the layer whose GEMM follows it
    shrink_calls = [c for c in log if c[0] == "lora_shrink"]
    shrink_ms = sum(d for n, d in launches if n == "lora_shrink")
    shrink_us = [d * 1e3 for n, d in launches if n == "lora_shrink"]
    assert len(shrink_calls) == len(shrink_us)
    shrink_shapes = {}
    for c, d in zip(shrink_calls, shrink_us):
        e = shrink_shapes.setdefault(tuple(c[1:4]), [0, 0.0])
        e[0] += 1
        e[1] += d
    shrink_rows = [{"M": M, "K": K, "R_padded": R, "launches": cnt, "avg_us": round(tot / cnt, 2)}
                   for (M, K, R), (cnt, tot) in sorted(shrink_shapes.items(), key=lambda kv: -kv[1][1])]
    n_layers = lambda c: c[5] if c[0] == "lora_linear_grouped" else 1
    rank_of = lambda c: true_rank if c[4] > 0 else 0
    keys_of = lambda c: c[7] if c[0] == "lora_linear_xattn" else 0      # attention inside the launch: 4 M N S more FLOPs
    call_flops = lambda c: n_layers(c) * lora_linear_flops(c[1], c[2], c[3], rank_of(c)) + 4.0 * c[1] * c[2] * keys_of(c)
    gemm_flops = sum(call_flops(c) for c in gemm_calls)
    gemm_total_ms = sum(gemm_ms) + shrink_ms
    attn_flops = sum(4.0 * c[1] * c[2] * c[3] * c[4] * c[5] for c in log if c[0] == "attention")
    step_flops = gemm_flops + attn_flops + conv_flops
    achieved_tf = gemm_flops / (gemm_total_ms * 1e-3) / 1e12
    by_shape = {}
    for c, d in zip(gemm_calls, gemm_ms):
        e = by_shape.setdefault(tuple(c[1:4]) + (rank_of(c), n_layers(c), keys_of(c)), [0, 0.0])
        e[0] += 1
        e[1] += d
    shape_rows = []
    for (M, N, K, R, G, S), (cnt, tot) in sorted(by_shape.items(), key=lambda kv: -kv[1][1]):
        fl = G * lora_linear_flops(M, N, K, R) + 4.0 * M * N * S
        tf = fl / (tot / cnt * 1e-3) / 1e12
        shape_rows.append({"M": M, "N": N, "K": K, "rank": R, "layers_per_launch": G, "launches": cnt,
                           "avg_us": round(tot / cnt * 1e3, 2), "ms_per_step": round(tot, 3), "tflops": round(tf, 1),
                           "frac": round(tf / PEAK_BF16_TFLOPS, 3)})
        if S:
            shape_rows[-1]["attention_keys_in_epilogue"] = S
    traffic, traffic_src = traffic_from_profiles("lora_gemm M2048 K1280 N10240")

    # ---- the other kernels of the path against their own rooflines ----------------------------------------------
    def pair(kernel_names, call_name, work_of):
        """(launch durations, algorithmic work) of one kernel family, matched in launch order with the call log."""
        durs = [d for n, d in launches if n in kernel_names]
        calls = [c for c in log if c[0] == call_name]
        per_call = len(kernel_names)
        assert len(durs) == per_call * len(calls), (call_name, len(durs), len(calls))
        return [(sum(durs[i * per_call:(i + 1) * per_call]), work_of(c), c) for i, c in enumerate(calls)]

    def gn_rows():
        """GroupNorm calls in call order: a full call owns the next statistics and the next apply launch, a call whose
        statistics came out of a convolution's epilogue owns the next apply launch only."""
        st = iter([d for n, d in launches if n == "group_norm_stats"])
        ap = iter([d for n, d in launches if n == "group_norm_apply"])
        rows = []
        for c in log:
            if c[0] == "group_norm":
                rows.append((next(st) + next(ap), 4.0 * c[1] * c[2] * c[3], c))
            elif c[0] == "group_norm_apply":
                rows.append((next(ap), 4.0 * c[1] * c[2] * c[3], c))
        assert next(st, None) is None and next(ap, None) is None
        return rows

    def roofline_rows(name, bound, rows, key_of):
        peak, unit, scale = (PEAK_BF16_TFLOPS, "TFLOP/s", 1e12) if bound == "mfma" else (PEAK_HBM_GBS, "GB/s", 1e9)
        tot_ms = sum(r[0] for r in rows)
        tot_work = sum(r[1] for r in rows)
        groups = {}
        for ms_, work, c in rows:
            e = groups.setdefault(key_of(c), [0, 0.0, 0.0])
            e[0] += 1; e[1] += ms_; e[2] += work
        ach = tot_work / (tot_ms * 1e-3) / scale if tot_ms > 0 else 0.0
        return {"kernel": name, "bound": bound, "achieved": round(ach, 1), "peak": peak, "unit": unit,
                "frac": round(ach / peak, 4), "launches_per_step": len(rows), "ms_per_step": round(tot_ms, 3),
                "by_shape": [{"shape": k, "launches": n, "avg_us": round(ms_ / n * 1e3, 2),
                              "achieved": round(w / (ms_ * 1e-3) / scale, 1), "frac": round(w / (ms_ * 1e-3) / scale / peak, 4)}
                             for k, (n, ms_, w) in sorted(groups.items(), key=lambda kv: -kv[1][1])[:6]]}

    rooflines = [
        roofline_rows("attention (kh_attention_bf16)", "mfma",
                      pair(("attention",), "attention", lambda c: 4.0 * c[1] * c[2] * c[3] * c[4] * c[5]),
                      lambda c: f"B{c[1]} H{c[2]} T{c[3]} S{c[4]}"),
        roofline_rows("conv3x3 implicit GEMM (kh_conv3x3_nhwc_bf16)", "mfma",
                      pair(("conv3x3",), "conv3x3", lambda c: 2.0 * c[1] * c[2] * c[3]),
                      lambda c: f"M{c[1]} Cout{c[2]} K{c[3]} stride{c[4]}"),
        roofline_rows("GroupNorm(+SiLU): statistics + apply launches (kh_group_norm_bf16), or the apply launch alone where the "
                      "convolution in front left the statistics (kh_group_norm_apply_bf16); bytes = one read + one write",
                      "hbm", gn_rows(), lambda c: f"N{c[1]} C{c[2]} HW{c[3]}" + (" (apply only)" if c[0] == "group_norm_apply" else "")),
        roofline_rows("LayerNorm (kh_layer_norm_bf16)", "hbm",
                      pair(("layer_norm",), "layer_norm", lambda c: 4.0 * c[1] * c[2]), lambda c: f"M{c[1]} D{c[2]}"),
        roofline_rows("ControlNet residual injection folded into the up-block concat (kh_concat_residual_bf16)", "hbm",
                      pair(("concat_residual",), "concat_residual",
                           lambda c: 2.0 * c[1] * (c[2] + c[3] * (1 + c[4]) + c[2] + c[3])),
                      lambda c: f"rows{c[1]} C{c[2]}+{c[3]}"),
    ]
    rooflines += sgmv_rooflines(dev)

    details = {"rooflines": rooflines, "lora_gemm_by_shape": shape_rows, "shrink_by_shape": shrink_rows,
               "traffic_note": "HBM-side bytes (read + written) of the largest launch as recorded in "
                               f"profiles/{PROFILE_SUMMARY.name} (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of `bench.py "
                               f"--kernel-probe`), not measured by this run; row: {traffic_src}"}
    short = lambda r: {k: r[k] for k in ("M", "N", "K", "launches", "avg_us", "ms_per_step", "frac")} | (
        {"xattn_keys": r["attention_keys_in_epilogue"]} if "attention_keys_in_epilogue" in r else {}) | (
        {"layers": r["layers_per_launch"]} if r["layers_per_launch"] > 1 else {})
    result = {
        "metric": "unet_step_ms_1024_2lora_1cn",
        "value": round(ms, 3),
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 3),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic (random-init SDXL UNet weights, seeded N(0,1) inputs, N(0,0.02) LoRA, N(0,0.1) residuals)",
        "config": {"workload": "SDXL UNet2DConditionModel step, latent [2,4,128,128] (1024x1024, CFG batch 2), "
                               "2 LoRAs (r64 s0.8 + r32 s0.6) on 722 linears, 1 ControlNet residual set, HIP graph",
                   "global_batch": 2, "parallelism": "single GPU"},
        "roofline": {"kernel": "LoRA linear GEMMs (lora_gemm_pipe / _wide / _ksplit: base GEMM + LoRA delta), all launches of "
                               "one step incl. the shrink launches",
                     "bound": "mfma", "achieved": round(achieved_tf, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved_tf / PEAK_BF16_TFLOPS, 4), "traffic": traffic,
                     "traffic_from": f"profiles/{PROFILE_SUMMARY.name} (largest launch; recorded, not measured by this run)",
                     "adapter_free_ms_per_step": round(ms_free, 3),
                     "lora_overhead_frac": round(ms / ms_free - 1.0, 4),
                     "rank_counted": true_rank,
                     "launches_per_step": len(gemm_ms), "shrink_launches_per_step": len(shrink_calls),
                     "shrink_ms_per_step": round(shrink_ms, 3), "gemm_ms_per_step": round(sum(gemm_ms), 3),
                     "avg_launch_us": round(gemm_total_ms / len(gemm_ms) * 1e3, 2),
                     "algorithmic_gflop_per_step": round(gemm_flops / 1e9, 1),
                     "step_tflop": round(step_flops / 1e12, 3), "output_finite": finite,
                     "by_shape": [short(r) for r in shape_rows[:9]]},
        "rooflines": [{k: r[k] for k in ("kernel", "bound", "achieved", "unit", "frac") if k in r} |
                      {k: r[k] for k in ("launches_per_step", "ms_per_step") if k in r} |
                      {"kernel": r["kernel"].split("(")[0].split(":")[0].strip()[:48]} |
                      ({"by_shape_frac": {(b["shape"].split(",")[0] + (" grouped" if "grouped" in b["shape"] else "")): b["frac"] for b in r["by_shape"][:4]}} if "by_shape" in r else {})
                      for r in rooflines],
        "kernel_ms_per_step": {k: round(v[1], 3) for k, v in sorted(by_kernel.items())},
    }
    if not args.no_cpu_baseline:
        cores = host_cores()
        t0 = time.perf_counter()
        full_s = cpu_baseline_full_step(cores)
        build_s = time.perf_counter() - t0 - full_s
        sec, sample_flops = cpu_baseline_sample(cores)
        est_ms = sec * 1e3 * step_flops / sample_flops
        print(f"bench.py: cpu baseline: model set-up {build_s:.1f} s, full step {full_s:.2f} s, mid-block sample {sec:.2f} s",
              file=sys.stderr)
        result["cpu_baseline"] = {"value": round(full_s * 1e3, 1), "unit": "ms", "cores": cores, "kind": "port",
                                  "cpu": cpu_model(), "host_cpus_visible": os.cpu_count(),
                                  "sample": f"ONE full step of the same workload on the fp32 oracle (2 LoRAs unmerged, 9 + 1 "
                                            f"residuals), {cores} threads, timed once without warm-up; cross-check: the UNet mid "
                                            f"block ({sample_flops / 1e12:.3f} TFLOP in {sec:.2f} s, median of 3) scaled by FLOPs "
                                            f"to the {step_flops / 1e12:.2f} TFLOP step = {est_ms:.0f} ms"}
        details["cpu_baseline_cross_check_ms"] = round(est_ms, 1)
    out_dir = ROOT / "gpurun_out"
    try:
        out_dir.mkdir(exist_ok=True)
        (out_dir / "bench_details.json").write_text(json.dumps(details, indent=1))
        result["details_file"] = "gpurun_out/bench_details.json"
    except OSError:
        pass
    print(json.dumps(result))


if __name__ == "__main__":
    main()
