#!/usr/bin/env python3
"""Benchmark of the Winograd 3x3 convolution hot path on one MI355X.

A step is one whole layer through the drop-in entry point (wino_conv: filter
transform + input transform + 16-way GEMM + output transform, inputs already in
HBM).  The default workload is the VGG-16 conv3-style layer the headline metric
is quoted on: 3x3, stride 1, pad 1, N=32, C=K=256, H=W=56, fp32, NCHW.

Prints ONE JSON line:
  value        effective TFLOP/s = 2*N*K*C*H*W*9 / t  (direct-convolution FLOP count)
  ms_per_step  ms per layer
  roofline     the dominant kernel (the batched GEMM, or the kernel containing it) timed with HIP
               events on the launch stream inside the library, against the dense MFMA peak
  cpu_baseline the oracle's fp32 OpenMP direct convolution on this host's cores (reported, not a target)
  stages       per-stage ms and achieved GB/s or TFLOP/s (extra, informative)
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# published MI355X peaks
HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"f32": 157.3, "f16": 2500.0, "bf16": 2500.0}

WORKLOADS = {
    # name: (N, C, K, H)
    "vgg16_conv3_N32_C256_K256_H56": (32, 256, 256, 56),
    "cfg1_N1_C64_K64_H56": (1, 64, 64, 56),
    "vgg16_conv4_N64_C512_K512_H28": (64, 512, 512, 28),
    "vgg16_conv5_N64_C512_K512_H14": (64, 512, 512, 14),
    "vgg16_conv1_2_N32_C64_K64_H224": (32, 64, 64, 224),
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="vgg16_conv3_N32_C256_K256_H56", choices=sorted(WORKLOADS))
    ap.add_argument("--layout", default="NCHW", choices=["NCHW", "NHWC", "CHWN"])
    ap.add_argument("--dtype", default="f32", choices=["f32", "f16", "bf16"])
    ap.add_argument("--algo", default="auto", choices=["auto", "staged", "epilogue", "fused"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this library runs one layer on ONE GPU; there is no multi-GPU path to measure "
              "(the batch would simply be split, no collective). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    from cudnntest_amd import ops, synth

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)

    N, C, K, H = WORKLOADS[args.workload]
    W = H
    layout = {"NCHW": ops.NCHW, "NHWC": ops.NHWC, "CHWN": ops.CHWN}[args.layout]
    tdt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[args.dtype]
    dt = {"f32": ops.F32, "f16": ops.F16, "bf16": ops.BF16}[args.dtype]
    algo = {"auto": ops.ALGO_AUTO, "staged": ops.ALGO_STAGED, "epilogue": ops.ALGO_EPILOGUE,
            "fused": ops.ALGO_FUSED}[args.algo]
    es = 4 if args.dtype == "f32" else 2

    x_h, w_h = synth.conv_inputs(N, C, K, H, W, seed=0x5EED, layout=layout)
    x = torch.from_numpy(x_h).cuda().to(tdt).contiguous()
    w = torch.from_numpy(w_h).cuda().to(tdt).contiguous()
    y = torch.empty(ops.act_shape(layout, N, K, H, W), dtype=tdt, device="cuda")

    def step():
        ops.conv(x, w, 1, layout, algo=algo, out=y)

    ops.warmup()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    # ---- timed region: exactly K steps -------------------------------------------------
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    direct_flops = 2.0 * N * K * C * H * W * 9
    value = direct_flops / (ms_per_step * 1e-3) / 1e12

    # ---- same steps again with the library's per-stage HIP events ------------------------
    ops.stage_timing(True)
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    st = ops.stage_times()
    ops.stage_timing(False)

    g = ops.geometry(dt, N, C, K, H, W, 1)
    P = g["P"]
    stage_ms = {k: (v[0] / v[1] if v[1] else None) for k, v in st.items()}
    gemm_flops = 2.0 * 16 * P * K * C
    alg_bytes = {
        "filter": (9 + 16) * K * C * es,
        "input": N * C * H * W * es + 16 * P * C * es,
        "output": 16 * P * K * 4 + N * K * H * W * es,
    }
    stages = {}
    for name in ("filter", "input", "output"):
        if stage_ms[name]:
            stages[name] = {"ms": round(stage_ms[name], 4),
                            "GBps": round(alg_bytes[name] / (stage_ms[name] * 1e-3) / 1e9, 1),
                            "frac_hbm": round(alg_bytes[name] / (stage_ms[name] * 1e-3) / 1e9 / HBM_PEAK_GBS, 3)}
    gemm_ms = stage_ms["gemm"]
    achieved = gemm_flops / (gemm_ms * 1e-3) / 1e12
    peak = MFMA_PEAK_TFLOPS[args.dtype]
    stages["gemm"] = {"ms": round(gemm_ms, 4), "TFLOPs": round(achieved, 2)}
    roofline = {"bound": "mfma", "kernel": "batched_gemm", "achieved": round(achieved, 2), "peak": peak,
                "unit": "TFLOP/s", "frac": round(achieved / peak, 4), "traffic": None}

    out = {
        "metric": "effective TFLOP/s (direct-conv FLOPs), VGG-16 3x3 layer, N=32",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": args.workload, "N": N, "C": C, "K": K, "H": H, "W": W, "pad": 1,
                   "layout": args.layout, "algo": args.algo, "winograd": "F(2x2,3x3)",
                   "filter_transform_in_step": True},
        "roofline": roofline,
        "stages": stages,
    }

    if not args.no_cpu_baseline:
        import oracle
        xs, ws = x_h, w_h
        if args.dtype != "f32":
            rnd = oracle.round_f16 if args.dtype == "f16" else oracle.round_bf16
            xs, ws = rnd(xs), rnd(ws)
        c0 = time.perf_counter()
        oracle.direct_conv_f32(xs, ws, 1, layout)
        c1 = time.perf_counter()
        out["cpu_baseline"] = {"value": round(direct_flops / (c1 - c0) / 1e12, 4), "unit": "TFLOP/s",
                               "cores": oracle.num_threads(), "kind": "port",
                               "sample": "the whole layer once (all N images), fp32 direct convolution, OpenMP",
                               "ms": round((c1 - c0) * 1e3, 1)}
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
