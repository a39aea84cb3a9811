#!/usr/bin/env python3
"""Benchmark of the Winograd 3x3 convolution hot path on one MI355X.

A step is one whole layer through the drop-in entry point (wino_conv: filter
transform + input transform + 16-way GEMM + output transform, or their fused
forms; inputs already in HBM).  The default workload is the VGG-16 conv3-style
layer the headline metric is quoted on: 3x3, stride 1, pad 1, N=32, C=K=256,
H=W=56, fp32, NCHW.  `--workload vgg16_all13` makes a step the thirteen VGG-16
convolutions (ReLU fused into the output stage) on synthetic activations of each
layer's shape; `--workload vgg16_stack` chains them through the conv-stack driver
(bias, ReLU and the five 2x2 poolings in the output stages, cached filter transforms).

Before the W warm-up steps the step runs untimed for --ramp-ms (200 ms): the GPU's clock governor needs
tens of milliseconds of load to reach its working frequency, and W steps of a 0.5 ms layer do not give it that.

Prints ONE JSON line:
  value        effective TFLOP/s = direct-convolution FLOPs (2*N*K*C*H*W*9) / time
  ms_per_step  ms per layer (per 13-layer pass for vgg16_all13)
  roofline     the dominant kernel -- the batched GEMM, or the kernel that contains it -- timed with
               HIP events recorded by the library on the launch stream, against the dense MFMA peak;
               algorithmic flops per launch = 2*16*P*K*C (2*36*P*K*C with --algo staged_f4); single-layer runs add
               the kernel's algorithmic bytes, flop/byte, min(MFMA peak, flop/byte x 8 TB/s) and its fraction of 8 TB/s
  cpu_baseline the oracle's fp32 OpenMP direct convolution on this host's cores (reported, not a target)
  stages       per-stage ms and achieved GB/s (algorithmic bytes) or TFLOP/s
  ms_per_step_filters_prepared   the same K steps with the filter bank transformed beforehand (single-layer runs)
  layout_transforms   the stand-alone permutations of the layer's input between its layout and the other two
               (wino_layout_transform; bytes = read + write), timed apart from the convolution
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
    # name: list of (N, C, K, H)
    "vgg16_conv3_N32_C256_K256_H56": [(32, 256, 256, 56)],
    "cfg1_N1_C64_K64_H56": [(1, 64, 64, 56)],
    "vgg16_conv4_N64_C512_K512_H28": [(64, 512, 512, 28)],
    "vgg16_conv5_N64_C512_K512_H14": [(64, 512, 512, 14)],
    "vgg16_conv1_2_N32_C64_K64_H224": [(32, 64, 64, 224)],
    "vgg16_all13": None,   # filled from synth.VGG16_CONV at N=32
    # the same thirteen layers as ONE stack (wino_stack_*): bias + ReLU in every output stage, 2x2 pooling after
    # conv 2, 4, 7, 10 and 13, activations handed from layer to layer, filter transforms cached outside the step
    "vgg16_stack": None,
    # the one shape the reference publishes latencies for (layoutTest/NHWC/result.num: NHWC, N=1..128)
    "ref_H22_C128_K128_N64": [(64, 128, 128, 22)],
    "ref_H22_C128_K128_N128": [(128, 128, 128, 22)],
}
# HBM bytes per launch of the dominant kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this
# script (summaries and the copy-kernel scale factor under profiles/), keyed by
# (workload, layout, dtype, resolved algo).
MEASURED_TRAFFIC = {
    # profiles/epilogue_fp32_nchw_vgg16_conv3_N32_hbm_traffic.txt: 596.1 MB fetched + 111.2 MB written (partial sums of the cut-up last round included)
    ("vgg16_conv3_N32_C256_K256_H56", "NCHW", "f32", "epilogue"): 707.3e6,
    # profiles/staged_fp32_nchw_vgg16_conv3_N32_hbm_traffic.txt: 449.1 MB fetched + 411.0 MB written
    ("vgg16_conv3_N32_C256_K256_H56", "NCHW", "f32", "staged"): 860.1e6,
    # profiles/fused_fp32_nchw_vgg16_conv1_2_N32_hbm_traffic.txt: 596.4 MB fetched + 411.0 MB written
    ("vgg16_conv1_2_N32_C64_K64_H224", "NCHW", "f32", "fused"): 1007.4e6,
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--workload", default="vgg16_conv3_N32_C256_K256_H56", choices=sorted(WORKLOADS))
    ap.add_argument("--layout", default="NCHW", choices=["NCHW", "NHWC", "CHWN"])
    ap.add_argument("--dtype", default="f32", choices=["f32", "f16", "bf16"])
    ap.add_argument("--algo", default="auto", choices=["auto", "staged", "epilogue", "fused", "staged_f4", "direct"])
    ap.add_argument("--batch", type=int, default=32, help="N of the vgg16_all13 / vgg16_stack workloads")
    ap.add_argument("--graph", action="store_true",
                    help="vgg16_stack: replay the pass from a HIP graph (one submission instead of ~30 launches)")
    ap.add_argument("--ramp-ms", type=float, default=200.0,
                    help="untimed steps before the warm-up, for this long: the shader clock needs tens of ms of "
                         "sustained load to leave its idle level (2.1 -> 2.4 GHz measured), more than W short steps give")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also launch a plain copy kernel of the first layer's input (known size) three times, so a "
                         "rocprofv3 --pmc run of this script can scale FETCH_SIZE / WRITE_SIZE")
    args = ap.parse_args()

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this library runs one layer on ONE GPU; there is no multi-GPU path to measure "
              "(the batch would simply be split, no collective). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch

    from cudnntest_amd import ops, synth

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)

    if args.graph and args.workload != "vgg16_stack":
        print("bench.py: --graph applies to --workload vgg16_stack", file=sys.stderr)
        sys.exit(2)
    layers = WORKLOADS[args.workload] or [(args.batch, C, K, H) for (C, K, H) in synth.VGG16_CONV]   # (N, C, K, H)
    multi = len(layers) > 1
    layout = {"NCHW": ops.NCHW, "NHWC": ops.NHWC, "CHWN": ops.CHWN}[args.layout]
    tdt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[args.dtype]
    dt = {"f32": ops.F32, "f16": ops.F16, "bf16": ops.BF16}[args.dtype]
    algo = {"auto": ops.ALGO_AUTO, "staged": ops.ALGO_STAGED, "epilogue": ops.ALGO_EPILOGUE,
            "fused": ops.ALGO_FUSED, "staged_f4": ops.ALGO_STAGED_F4, "direct": ops.ALGO_DIRECT}[args.algo]
    es = 4 if args.dtype == "f32" else 2

    stack = None
    if args.workload == "vgg16_stack":
        if args.algo == "staged_f4":
            print("bench.py: the stack driver has no F(4x4,3x3) mode", file=sys.stderr)
            sys.exit(2)
        pools = {1, 3, 6, 9, 12}
        descs = [dict(K=K, layout_in=layout, layout_out=layout, relu=True, pool=i in pools, algo=algo)
                 for i, (N, C, K, H) in enumerate(layers)]
        stack = ops.ConvStack(tdt, args.batch, 3, 224, 224, descs)
        for i, (N, C, K, H) in enumerate(layers):
            _, w_h = synth.conv_inputs(1, C, K, 4, 4, seed=0x5EED + i, layout=layout)
            b_h = synth.normal(K, 0xB1A5 + i, 0.05)
            stack.set_layer(i, torch.from_numpy(w_h).cuda().to(tdt).contiguous(), torch.from_numpy(b_h).float().cuda().to(tdt))
    tensors, host_inputs = [], []
    for i, (N, C, K, H) in enumerate(layers):
        if stack is not None and i > 0:
            break
        x_h, w_h = synth.conv_inputs(N, C, K, H, H, seed=0x5EED + i, layout=layout)
        x = torch.from_numpy(x_h).cuda().to(tdt).contiguous()
        w = torch.from_numpy(w_h).cuda().to(tdt).contiguous()
        y = torch.empty(ops.act_shape(layout, N, K, H, H), dtype=tdt, device="cuda")
        tensors.append((x, w, y))
        if i == 0:
            host_inputs = (x_h, w_h)

    stack_out = torch.empty(stack.out_shape, dtype=tdt, device="cuda") if stack is not None else None

    def step():
        if stack is not None:
            stack.forward(tensors[0][0], out=stack_out, graph=args.graph)
            return
        for (x, w, y) in tensors:
            ops.conv(x, w, 1, layout, algo=algo, relu=multi, out=y)

    ops.warmup()
    if args.copy_probe:
        for _ in range(3):
            ops.layout_transform(tensors[0][0], layout, layout)   # same layout both sides: a plain copy
    t_ramp = time.perf_counter()
    while (time.perf_counter() - t_ramp) * 1e3 < args.ramp_ms:
        for _ in range(10):
            step()
        torch.cuda.synchronize()
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
    direct_flops = sum(2.0 * N * K * C * H * H * 9 for (N, C, K, H) in layers)
    value = direct_flops / (ms_per_step * 1e-3) / 1e12

    # ---- the same K steps again, the library bracketing every stage with HIP events --------
    ops.stage_timing(True)
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    st = ops.stage_stats()
    ops.stage_timing(False)

    per_step = {k: (v[0] / args.steps) for k, v in st.items()}        # ms per step, summed over layers
    gemm_flops = alg_in = alg_out = alg_flt = 0.0
    resolved = []
    for (N, C, K, H) in layers:
        a = ops.pick_algo(layout, dt, N, C, K, H, H) if algo == ops.ALGO_AUTO else algo
        f4 = a == ops.ALGO_STAGED_F4
        g = ops.f4_geometry(dt, N, C, K, H, H, 1) if f4 else ops.geometry(dt, N, C, K, H, H, 1)
        P, nxi = g["P"], (36 if f4 else 16)
        resolved.append(ops.ALGO_NAMES[a])
        if a == ops.ALGO_DIRECT:                  # no Winograd: the direct-convolution flops, no transforms
            gemm_flops += 2.0 * N * K * C * H * H * 9
            continue
        gemm_flops += 2.0 * nxi * P * K * C
        if stack is None:
            alg_flt += (9 + nxi) * K * C * es
        if a != ops.ALGO_FUSED:
            alg_in += N * C * H * H * es + nxi * P * C * es
        if a in (ops.ALGO_STAGED, ops.ALGO_STAGED_F4):
            pooled = stack is not None and len(resolved) - 1 in (1, 3, 6, 9, 12)
            alg_out += nxi * P * K * 4 + N * K * H * H * es // (4 if pooled else 1)
    stages = {}
    for name, nbytes in (("filter", alg_flt), ("input", alg_in), ("output", alg_out)):
        if per_step[name] > 0 and nbytes > 0:
            gbs = nbytes / (per_step[name] * 1e-3) / 1e9
            stages[name] = {"ms": round(per_step[name], 4), "GBps": round(gbs, 1),
                            "frac_hbm": round(gbs / HBM_PEAK_GBS, 3)}
            if not multi:                          # one span per step: shortest and longest of the K steps
                stages[name].update(min_ms=round(st[name][1], 4), max_ms=round(st[name][2], 4))
    gemm_ms = per_step["gemm"]
    achieved = gemm_flops / (gemm_ms * 1e-3) / 1e12
    peak = MFMA_PEAK_TFLOPS[args.dtype]
    stages["gemm"] = {"ms": round(gemm_ms, 4), "TFLOPs": round(achieved, 2)}
    if not multi:
        stages["gemm"].update(min_ms=round(st["gemm"][1], 4), max_ms=round(st["gemm"][2], 4))
    kernel = {"staged": "gemm_128x128_kernel", "epilogue": "gemm_rows_kernel", "fused": "fused_rows_kernel",
              "staged_f4": "gemm_128x128_kernel",
              "direct": "direct_small_c_kernel" if args.dtype == "f32" else "direct_small_c16_kernel"}
    algo_label = resolved[0] if len(set(resolved)) == 1 else "mixed"
    traffic = MEASURED_TRAFFIC.get((args.workload, args.layout, args.dtype, algo_label))
    roofline = {"bound": "mfma", "kernel": kernel.get(algo_label, "per-layer choice"),
                "achieved": round(achieved, 2), "peak": peak, "unit": "TFLOP/s",
                "frac": round(achieved / peak, 4), "traffic": traffic,
                "flops_per_launch": gemm_flops if not multi else None}

    N0, C0, K0, H0 = layers[0]
    if not multi:
        # the dominant kernel's algorithmic bytes, its arithmetic intensity, and what the two roofs allow together
        Pn = ops.geometry(dt, N0, C0, K0, H0, H0, 1)["P"]
        xb, yb = N0 * C0 * H0 * H0 * es, N0 * K0 * H0 * H0 * es
        kb = {"staged": 16 * Pn * C0 * es + 16 * K0 * C0 * es + 16 * Pn * K0 * 4,
              "epilogue": 16 * Pn * C0 * es + 16 * K0 * C0 * es + yb,
              "fused": xb + 16 * K0 * C0 * es + yb,
              "direct": xb + 9 * K0 * C0 * es + yb}.get(algo_label)
        if kb:
            ai = gemm_flops / kb
            gbs = kb / (gemm_ms * 1e-3) / 1e9
            roofline.update(algorithmic_bytes=kb, flop_per_byte=round(ai, 1),
                            attainable=round(min(peak, ai * HBM_PEAK_GBS / 1e3), 1),
                            frac_hbm=round(gbs / HBM_PEAK_GBS, 3))
            if ai * HBM_PEAK_GBS / 1e3 < peak:
                # the memory roof is the lower one for this kernel and type: it is the bound that is reported
                roofline.update(bound="hbm", achieved=round(gbs, 1), peak=HBM_PEAK_GBS, unit="GB/s",
                                frac=round(gbs / HBM_PEAK_GBS, 4), mfma_achieved=round(achieved, 2),
                                mfma_frac=round(achieved / peak, 4))
    out = {
        "metric": "effective TFLOP/s (direct-conv FLOPs), VGG-16 3x3 layer, N=32",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": args.workload, "layers": len(layers), "N": N0, "C": C0, "K": K0, "H": H0, "W": H0,
                   "pad": 1, "layout": args.layout, "algo": args.algo, "resolved_algo": resolved,
                   "winograd": "F(4x4,3x3)" if algo_label == "staged_f4" else "F(2x2,3x3)",
                   "filter_transform_in_step": stack is None, "relu": multi,
                   "bias_and_pooling_in_step": stack is not None, "hip_graph": args.graph},
        "roofline": roofline,
        "stages": stages,
    }

    # ---- the same K steps with the filter bank transformed beforehand (filter transform excluded) ----
    if not multi and stack is None and resolved[0] in ("staged", "epilogue", "fused"):
        x0, w0, y0 = tensors[0]
        U0 = ops.filter_transform(w0, layout)
        a0 = {"staged": ops.ALGO_STAGED, "epilogue": ops.ALGO_EPILOGUE, "fused": ops.ALGO_FUSED}[resolved[0]]
        for _ in range(args.warmup):
            ops.conv_prepared(x0, U0, K0, 1, layout, algo=a0, out=y0)
        torch.cuda.synchronize()
        tp = time.perf_counter()
        for _ in range(args.steps):
            ops.conv_prepared(x0, U0, K0, 1, layout, algo=a0, out=y0)
        torch.cuda.synchronize()
        out["ms_per_step_filters_prepared"] = round((time.perf_counter() - tp) * 1e3 / args.steps, 4)

    # ---- the stand-alone layout permutations of the layer's input, timed separately ------------
    if not multi and stack is None:
        names = {ops.NCHW: "NCHW", ops.NHWC: "NHWC", ops.CHWN: "CHWN"}
        x0 = tensors[0][0]
        perms = {}
        for dst_l in (ops.NCHW, ops.NHWC, ops.CHWN):
            if dst_l == layout:
                continue
            x1 = ops.layout_transform(x0, layout, dst_l)
            for (a, la, lb) in ((x0, layout, dst_l), (x1, dst_l, layout)):
                for _ in range(3):
                    ops.layout_transform(a, la, lb)
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(20):
                    ops.layout_transform(a, la, lb)
                e1.record()
                torch.cuda.synchronize()
                ms = e0.elapsed_time(e1) / 20
                gbs = 2.0 * x0.numel() * es / (ms * 1e-3) / 1e9
                perms[f"{names[la]}->{names[lb]}"] = {"ms": round(ms, 4), "GBps": round(gbs, 1),
                                                      "frac_hbm": round(gbs / HBM_PEAK_GBS, 3)}
            del x1
        out["layout_transforms"] = perms

    if not args.no_cpu_baseline:
        import oracle
        xs, ws = host_inputs
        if args.dtype != "f32":
            rnd = oracle.round_f16 if args.dtype == "f16" else oracle.round_bf16
            xs, ws = rnd(xs), rnd(ws)
        N, C, K, H = layers[0]
        fl = 2.0 * N * K * C * H * H * 9
        c0 = time.perf_counter()
        oracle.direct_conv_f32(xs, ws, 1, layout, relu=multi)
        c1 = time.perf_counter()
        out["cpu_baseline"] = {"value": round(fl / (c1 - c0) / 1e12, 4), "unit": "TFLOP/s",
                               "cores": oracle.num_threads(), "kind": "port",
                               "sample": ("the whole layer once (all N images)" if not multi else
                                          "the first of the 13 layers once (all N images, convolution and ReLU)") +
                                         ", fp32 direct convolution, OpenMP",
                               "ms": round((c1 - c0) * 1e3, 1)}
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
