#!/usr/bin/env python3
"""Benchmark of the adapter-augmented SDXL UNet step on one MI355X.

Workload (BASELINE.json configs[2], the configuration the metric is quoted on): one bf16
UNet2DConditionModel denoising step, random-init SDXL weights, latent [2,4,128,128] (CFG batch 2,
1024x1024), t=500, context [2,77,2048], pooled text [2,1280], time_ids [2,6]; two LoRAs (rank 64 scale
0.8, rank 32 scale 0.6) on all 722 attention / feed-forward / projection linears, one ControlNet
residual set (9 down + 1 mid, ~N(0,0.1)).  A step = one HIP-graph replay of the whole forward, inputs
resident in HBM.

Prints ONE JSON line: ms per step (value), the adapter-free step beside it, a `roofline` object for the
dominant kernel (the fused LoRA GEMM: algorithmic FLOPs of all its launches in a step / the sum of their
durations, each launch timed with its own HIP event pair on the launch stream) and a `cpu_baseline`
object (the fp32 CPU oracle timed on a bounded sample and scaled by FLOPs).
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


def add_random_loras(unet, device, specs=(("r64", 64, 0.8), ("r32", 32, 0.6)), seed=10):
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


def cpu_baseline(cores):
    """fp32 CPU oracle on a bounded sample: the UNet mid block (resnet, 10 transformer blocks with both
    LoRAs, resnet; batch 2, 32x32 latent) -- scaled to a whole step by algorithmic FLOPs."""
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
        for _ in range(3):
            t0 = time.perf_counter()
            blk(x, temb, ctx)
            ts.append(time.perf_counter() - t0)
    ts.sort()
    return ts[1], flops


# HBM-side bytes of the largest LoRA GEMM launch, measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on
# `bench.py --traffic-probe` and calibrated against a copy of known size (summary under profiles/)
GEMM_TRAFFIC_BYTES = 164.7e6


def traffic_probe():
    """Counter calibration run: a device copy of known size (64 MiB read + 64 MiB written), then the largest
    LoRA linear of the step (GEGLU projection, M 2048, K 1280, N 10240, packed rank 128) as shrink + GEMM,
    three times.  Under `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` the copy gives the factor between
    the counter and bytes; the GEMM rows give its HBM traffic per launch."""
    import torch
    from katz_amd import ops

    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(0)
    src = torch.randn(16 << 20, device=dev, generator=g)            # 64 MiB fp32
    dst = torch.empty_like(src)
    M, K, N, R = 2048, 1280, 10240, 128
    x = torch.randn(M, K, device=dev, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, device=dev, generator=g) * 0.02).to(torch.bfloat16)
    b = torch.randn(N, device=dev, generator=g).to(torch.bfloat16)
    a_cat = (torch.randn(R, K, device=dev, generator=g) * 0.02).to(torch.bfloat16)
    b_cat = (torch.randn(N, R, device=dev, generator=g) * 0.02).to(torch.bfloat16)
    scale = torch.full((R,), 0.8, device=dev)
    torch.cuda.synchronize()
    for _ in range(3):
        dst.copy_(src)
        t = ops.lora_shrink(x, a_cat, scale)
        ops.lora_linear_pre(x, w, b, t, b_cat, geglu=True)
    torch.cuda.synchronize()
    print(json.dumps({"traffic_probe": {"copy_bytes_read": src.numel() * 4, "copy_bytes_written": src.numel() * 4,
                                        "gemm": {"M": M, "N": N, "K": K, "R": R, "geglu": True},
                                        "algorithmic_bytes": 2 * (M * K + K * N + M * N // 2 + R * (K + N))}}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="run only a 64 MiB copy and the dominant LoRA GEMM shape a few times (for rocprofv3 --pmc)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU only (no collectives, no sharding); --gpus must be 1",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from katz_amd.graph import GraphedUNetStep

    if args.traffic_probe:
        traffic_probe()
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

    # per-kernel accounting of the instrumented step
    by_kernel = {}
    for name, dur in launches:
        e = by_kernel.setdefault(name, [0, 0.0])
        e[0] += 1
        e[1] += dur
    gemm_calls = [c for c in log if c[0] in ("lora_linear", "lora_linear_grouped")]
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
    shrink_rows = [{"M": M, "K": K, "R": R, "launches": cnt, "avg_us": round(tot / cnt, 2)}
                   for (M, K, R), (cnt, tot) in sorted(shrink_shapes.items(), key=lambda kv: -kv[1][1])]
    n_layers = lambda c: c[5] if c[0] == "lora_linear_grouped" else 1
    gemm_flops = sum(n_layers(c) * lora_linear_flops(c[1], c[2], c[3], c[4]) for c in gemm_calls)
    gemm_total_ms = sum(gemm_ms) + shrink_ms
    attn_flops = sum(4.0 * c[1] * c[2] * c[3] * c[4] * c[5] for c in log if c[0] == "attention")
    step_flops = gemm_flops + attn_flops + conv_flops
    achieved_tf = gemm_flops / (gemm_total_ms * 1e-3) / 1e12
    # the largest fused-LoRA GEMM shape class, for the headline "fused LoRA-GEMM TFLOP/s"
    by_shape = {}
    for c, d in zip(gemm_calls, gemm_ms):
        e = by_shape.setdefault(tuple(c[1:5]) + (n_layers(c),), [0, 0.0])
        e[0] += 1
        e[1] += d
    shape_rows = []
    for (M, N, K, R, G), (cnt, tot) in sorted(by_shape.items(), key=lambda kv: -kv[1][1]):
        fl = G * lora_linear_flops(M, N, K, R)
        shape_rows.append({"M": M, "N": N, "K": K, "R": R, "layers_per_launch": G, "launches": cnt, "avg_us": round(tot / cnt * 1e3, 2),
                           "tflops": round(fl / (tot / cnt * 1e-3) / 1e12, 1)})

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
        "adapter_free_ms_per_step": round(ms_free, 3),
        "lora_overhead_frac": round(ms / ms_free - 1.0, 4),
        "step_tflop": round(step_flops / 1e12, 3),
        "step_tflops_per_s": round(step_flops / (ms * 1e-3) / 1e12, 1),
        "output_finite": finite,
        "roofline": {"kernel": "lora_gemm_kernel (fused base GEMM + LoRA delta, all launches of one step)",
                     "bound": "mfma", "achieved": round(achieved_tf, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved_tf / PEAK_BF16_TFLOPS, 4), "traffic": GEMM_TRAFFIC_BYTES,
                     "traffic_note": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of `bench.py --traffic-probe`, largest launch "
                                     "(M 2048, K 1280, N 10240, R 128): 143.7 MB read + 21.0 MB written; algorithmic 55.4 MB",
                     "launches_per_step": len(gemm_ms), "shrink_launches_per_step": len(shrink_calls),
                     "shrink_ms_per_step": round(shrink_ms, 3), "avg_launch_us": round(gemm_total_ms / len(gemm_ms) * 1e3, 2),
                     "algorithmic_gflop_per_step": round(gemm_flops / 1e9, 1), "by_shape": shape_rows[:8],
                     "shrink_by_shape": shrink_rows[:6]},
        "kernel_ms_per_step": {k: {"launches": v[0], "ms": round(v[1], 3)} for k, v in sorted(by_kernel.items())},
    }
    if not args.no_cpu_baseline:
        cores = min(16, os.cpu_count() or 1)
        sec, sample_flops = cpu_baseline(cores)
        est_ms = sec * 1e3 * step_flops / sample_flops
        result["cpu_baseline"] = {"value": round(est_ms, 1), "unit": "ms", "cores": cores, "kind": "port",
                                  "sample": f"fp32 oracle, UNet mid block (2 resnets + 10 transformer blocks with both "
                                            f"LoRAs, batch 2, 32x32) = {sample_flops / 1e12:.3f} TFLOP in {sec:.2f} s, "
                                            f"scaled by FLOPs to the {step_flops / 1e12:.2f} TFLOP step"}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
