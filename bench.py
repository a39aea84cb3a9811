#!/usr/bin/env python3
"""Benchmark of the Winograd 3x3 convolution hot path on one MI355X.

A step is one whole layer through the drop-in entry point (wino_conv: filter
transform + input transform + 16- or 36-way GEMM + output transform, or their fused
forms, as the library's automatic choice resolves; inputs already in HBM).  The default workload is the VGG-16 conv3-style
layer the headline metric is quoted on: 3x3, stride 1, pad 1, N=32, C=K=256,
H=W=56, fp32, NCHW.  `--workload vgg16_all13` makes a step the thirteen VGG-16
convolutions (ReLU fused into the output stage) on synthetic activations of each
layer's shape; `--workload vgg16_stack` chains them through the conv-stack driver
(bias, ReLU and the five 2x2 poolings in the output stages, cached filter transforms).

Before the W warm-up steps the step runs untimed for --ramp-ms (200 ms): the GPU's clock governor needs
tens of milliseconds of load to reach its working frequency, and W steps of a 0.5 ms layer do not give it that.

Prints ONE JSON line:
  ms_per_step  the MEDIAN of the K steps' own durations (an event on the launch stream after every step), ms per layer
               (per 13-layer pass for vgg16_all13); ms_per_step_wall_mean is host wall time over the same K steps / K
  value        effective TFLOP/s = direct-convolution FLOPs (2*N*K*C*H*W*9) / ms_per_step
  roofline     the dominant kernel -- the batched GEMM, or the kernel that contains it -- timed with
               HIP events recorded by the library on the launch stream, against the dense MFMA peak;
               algorithmic flops per launch = 2*16*P*K*C (2*36*P*K*C with --algo staged_f4, the direct-convolution count
               for the direct kernels); single-layer runs add the kernel's algorithmic bytes, flop/byte,
               min(MFMA peak, flop/byte x 8 TB/s) and its fraction of 8 TB/s; traffic = HBM bytes per launch
               measured with rocprofv3 --pmc (traffic_source names the summary under profiles/), null where
               no such run is committed
  cpu_baseline the oracle's fp32 OpenMP direct convolution on this host's cores (reported, not a target)
  configs_summary   the LAST key of the line: every entry of `configs` as [ms, effective TFLOP/s, pipeline, fraction of
               what the two roofs allow], so that a record which keeps only the line's tail still holds them all
  stages       per-stage ms and achieved GB/s (algorithmic bytes) or TFLOP/s
  ms_per_step_filters_prepared   the same K steps with the filter bank transformed beforehand (single-layer runs)
  layout_transforms   the stand-alone permutations of the layer's input between its layout and the other two
               (wino_layout_transform; bytes = read + write), timed apart from the convolution
  configs      (default workload only, after its timed region) the other benchmark configurations, a few steps
               each: ms (median), effective TFLOP/s, the dominant kernel with its fraction of the MFMA peak and of
               min(MFMA peak, flop/byte x 8 TB/s); for the 13-layer f16 / bf16 passes also per layer
               configs.reference_published_sweep: the reference's only committed latencies (NHWC, H=22, C=K=128,
               N = 1 .. 128, layoutTest/NHWC/result.num) beside this library's, timed as the reference timed them
"""
import argparse
import json
import os
import statistics
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
# script (the summary file holds the counters and the copy-kernel scale factor), keyed by
# (workload, layout, dtype, resolved algo): (bytes, summary under profiles/).
MEASURED_TRAFFIC = {
    # the GEMM of the F(4x4) pipeline (gemm_128x128_walk_spread_kernel): 320.8 MB fetched + 231.2 MB written
    ("vgg16_conv3_N32_C256_K256_H56", "NCHW", "f32", "staged_f4"):
        (552.1e6, "profiles/staged_f4_fp32_nchw_vgg16_conv3_N32_counters.txt"),
    ("vgg16_conv3_N32_C256_K256_H56", "NHWC", "f32", "staged_f4"):
        (554.3e6, "profiles/staged_f4_fp32_nhwc_vgg16_conv3_N32_counters.txt"),   # 323.1 MB fetched + 231.2 MB written
    # gemm_rows_f4_kernel: 1435.0 MB fetched (a patch's rows of V once per filter tile, most of it from the L2) + 515.0 MB written
    ("vgg16_conv3_N32_C256_K256_H56", "NCHW", "f32", "epilogue_f4"):
        (1949.9e6, "profiles/epilogue_f4_fp32_nchw_vgg16_conv3_N32_counters.txt"),
    # gemm_rows_kernel (partial sums of the cut-up last round included)
    ("vgg16_conv3_N32_C256_K256_H56", "NCHW", "f32", "epilogue"):
        (746.9e6, "profiles/epilogue_fp32_nchw_vgg16_conv3_N32_counters.txt"),
    ("vgg16_conv3_N32_C256_K256_H56", "NCHW", "f32", "staged"):
        (896.8e6, "profiles/staged_fp32_nchw_vgg16_conv3_N32_counters.txt"),
    ("vgg16_conv1_2_N32_C64_K64_H224", "NCHW", "f32", "fused"):
        (994.6e6, "profiles/fused_fp32_nchw_vgg16_conv1_2_N32_counters.txt"),
    # direct16_rows_kernel: 93.6 + 51.4 MB
    ("vgg16_conv3_N32_C256_K256_H56", "NCHW", "bf16", "direct"):
        (145.0e6, "profiles/direct16_rows_bf16_nchw_vgg16_conv3_N32_counters.txt"),
    ("vgg16_conv1_2_N32_C64_K64_H224", "NCHW", "bf16", "direct"):
        (533.6e6, "profiles/direct16_rows_bf16_nchw_vgg16_conv1_2_N32_counters.txt"),
    # the same kernel from NHWC tensors, and from CHWN ones (one image of width W * N: 4-row blocks read 6 input rows)
    ("vgg16_conv3_N32_C256_K256_H56", "NHWC", "bf16", "direct"):
        (145.7e6, "profiles/direct16_rows_bf16_nhwc_vgg16_conv3_N32_counters.txt"),
    ("vgg16_conv3_N32_C256_K256_H56", "CHWN", "bf16", "direct"):
        (235.0e6, "profiles/direct16_rows_bf16_chwn_vgg16_conv3_N32_counters.txt"),
    # gemm_rows_kernel in bf16
    ("vgg16_conv3_N32_C256_K256_H56", "NCHW", "bf16", "epilogue"):
        (328.4e6, "profiles/epilogue_bf16_nchw_vgg16_conv3_N32_counters.txt"),
}
# what the default run also times, after the headline's timed region: (name, workload, dtype, layout)
OTHER_CONFIGS = [
    ("cfg1_N1_C64_K64_H56_f32", "cfg1_N1_C64_K64_H56", "f32", "NCHW"),
    ("cfg2_N32_C256_K256_H56_f32_NHWC", "vgg16_conv3_N32_C256_K256_H56", "f32", "NHWC"),
    ("cfg2_N32_C256_K256_H56_f32_CHWN", "vgg16_conv3_N32_C256_K256_H56", "f32", "CHWN"),
    ("cfg3a_N64_C512_K512_H28_f32", "vgg16_conv4_N64_C512_K512_H28", "f32", "NCHW"),
    ("cfg3b_N64_C512_K512_H14_f32", "vgg16_conv5_N64_C512_K512_H14", "f32", "NCHW"),
    ("cfg4_N32_C64_K64_H224_f32", "vgg16_conv1_2_N32_C64_K64_H224", "f32", "NCHW"),
    ("cfg5_vgg16_all13_N32_f16", "vgg16_all13", "f16", "NCHW"),
    ("cfg5_vgg16_all13_N32_bf16", "vgg16_all13", "bf16", "NCHW"),
    ("cfg5_vgg16_all13_N32_bf16_NHWC", "vgg16_all13", "bf16", "NHWC"),
    ("cfg5_vgg16_all13_N32_bf16_CHWN", "vgg16_all13", "bf16", "CHWN"),
]
KERNEL_OF = {"epilogue_f4": "gemm_rows_f4_kernel", "staged": "gemm_128x128_kernel / gemm_128x128_walk_kernel / gemm_128x128_walk_spread_kernel", "epilogue": "gemm_rows_kernel", "fused": "fused_rows_kernel",
             "staged_f4": "gemm_128x128_walk_spread_kernel / gemm_128x128_kernel", "direct": "direct16_rows_kernel / direct_small_c kernel / direct_few_pixels_kernel"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--workload", default="vgg16_conv3_N32_C256_K256_H56", choices=sorted(WORKLOADS))
    ap.add_argument("--layout", default="NCHW", choices=["NCHW", "NHWC", "CHWN"])
    ap.add_argument("--dtype", default="f32", choices=["f32", "f16", "bf16"])
    ap.add_argument("--algo", default="auto", choices=["auto", "staged", "epilogue", "fused", "staged_f4", "direct", "epilogue_f4"])
    ap.add_argument("--shape", default=None, metavar="N,C,K,H",
                    help="a single layer of this shape instead of a named workload (kernel experiments)")
    ap.add_argument("--batch", type=int, default=32, help="N of the vgg16_all13 / vgg16_stack workloads")
    ap.add_argument("--graph", action="store_true",
                    help="vgg16_stack: replay the pass from a HIP graph (one submission instead of ~30 launches)")
    ap.add_argument("--ramp-ms", type=float, default=200.0,
                    help="untimed steps before the warm-up, for this long: the shader clock needs tens of ms of "
                         "sustained load to leave its idle level (2.1 -> 2.4 GHz measured), more than W short steps give")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="default workload: skip the `configs` object (the other benchmark configurations)")
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
    LAYOUT = {"NCHW": ops.NCHW, "NHWC": ops.NHWC, "CHWN": ops.CHWN}
    TDT = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}
    DT = {"f32": ops.F32, "f16": ops.F16, "bf16": ops.BF16}
    ALGO = {"auto": ops.ALGO_AUTO, "staged": ops.ALGO_STAGED, "epilogue": ops.ALGO_EPILOGUE,
            "fused": ops.ALGO_FUSED, "staged_f4": ops.ALGO_STAGED_F4, "direct": ops.ALGO_DIRECT,
            "epilogue_f4": ops.ALGO_EPILOGUE_F4}

    if args.shape:
        WORKLOADS["custom"] = [tuple(int(v) for v in args.shape.split(","))]
        args.workload = "custom"

    def layers_of(workload):
        return WORKLOADS[workload] or [(args.batch, C, K, H) for (C, K, H) in synth.VGG16_CONV]   # (N, C, K, H)

    def timed(step, steps, warmup, group=1):
        """(median ms per step, wall-clock mean ms per step) of exactly `steps` steps after `warmup`.  An event is
        recorded on the launch stream after every `group` steps and the median is taken over those spans (group > 1
        for steps of a few tens of microseconds, where an event between two launches would be part of what is timed)."""
        for _ in range(warmup):
            step()
        spans = steps // group
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(spans + 1)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ev[0].record()
        for i in range(spans):
            for _ in range(group):
                step()
            ev[i + 1].record()
        for _ in range(steps - spans * group):
            step()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        per = [ev[i].elapsed_time(ev[i + 1]) / group for i in range(spans)]
        return statistics.median(per), (t1 - t0) * 1e3 / steps

    def staged_pass(step, steps):
        """per-stage (sum, min, max, spans) of `steps` more steps, the library bracketing every stage with events"""
        ops.stage_timing(True)
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        st = ops.stage_stats()
        ops.stage_timing(False)
        return st

    def kernel_roofline(layout, dtype, a, N, C, K, H, gemm_ms):
        """the dominant kernel of one layer against both roofs"""
        dt, es, peak = DT[dtype], (4 if dtype == "f32" else 2), MFMA_PEAK_TFLOPS[dtype]
        name = ops.ALGO_NAMES[a]
        f4 = a in (ops.ALGO_STAGED_F4, ops.ALGO_EPILOGUE_F4)
        g = ops.f4_geometry(dt, N, C, K, H, H, 1) if f4 else ops.geometry(dt, N, C, K, H, H, 1)
        P, nxi = g["P"], (36 if f4 else 16)
        xb, yb = N * C * H * H * es, N * K * H * H * es
        flops = 2.0 * N * K * C * H * H * 9 if a == ops.ALGO_DIRECT else 2.0 * nxi * P * K * C
        kb = {"staged": nxi * P * C * es + nxi * K * C * es + nxi * P * K * 4,
              "staged_f4": nxi * P * C * es + nxi * K * C * es + nxi * P * K * 4,
              "epilogue": 16 * P * C * es + 16 * K * C * es + yb,
              "epilogue_f4": 36 * P * C * es + 36 * K * C * es + yb,
              "fused": xb + 16 * K * C * es + yb,
              "direct": xb + 9 * K * C * es + yb}[name]
        ai = flops / kb
        attainable = min(peak, ai * HBM_PEAK_GBS / 1e3)
        achieved = flops / (gemm_ms * 1e-3) / 1e12
        return {"algo": name, "kernel": KERNEL_OF[name], "kernel_ms": round(gemm_ms, 4), "flops": flops,
                "algorithmic_bytes": kb, "flop_per_byte": round(ai, 1), "achieved_tflops": round(achieved, 2),
                "frac_mfma": round(achieved / peak, 4), "attainable_tflops": round(attainable, 1),
                "frac_of_attainable": round(achieved / attainable, 4),
                "bound": "mfma" if attainable >= peak else "hbm",
                "GBps": round(kb / (gemm_ms * 1e-3) / 1e9, 1)}

    def device_tensors(layers, layout, dtype, seed):
        """x, w, y of every layer, generated on the device (seeded): uniform[-1, 1) activations, N(0, sqrt(2/(9C))) filters"""
        g = torch.Generator(device="cuda").manual_seed(seed)
        out = []
        for (N, C, K, H) in layers:
            x = (torch.rand(ops.act_shape(layout, N, C, H, H), device="cuda", generator=g) * 2 - 1).to(TDT[dtype])
            wshape = {ops.NCHW: (K, C, 3, 3), ops.NHWC: (K, 3, 3, C), ops.CHWN: (C, 3, 3, K)}[layout]
            w = (torch.randn(wshape, device="cuda", generator=g) * (2.0 / (9 * C)) ** 0.5).to(TDT[dtype])
            y = torch.empty(ops.act_shape(layout, N, K, H, H), dtype=TDT[dtype], device="cuda")
            out.append((x, w, y))
        return out

    def other_config(workload, dtype, layout_name="NCHW"):
        """one of the other benchmark configurations, the automatic choice of pipeline: a few steps"""
        layout, layers = LAYOUT[layout_name], layers_of(workload)
        many = len(layers) > 1
        tens = device_tensors(layers, layout, dtype, 0xBE7C)

        def run(sel):
            for (x, w, y) in sel:
                ops.conv(x, w, 1, layout, relu=many, out=y)
        tiny = layers[0][0] == 1                      # N = 1: a step is a few tens of microseconds
        steps = 20 if many else (200 if tiny else 30)
        # generating the tensors left the GPU idle: untimed steps for 100 ms bring the clock back up, as before the headline
        r0 = time.perf_counter()
        while time.perf_counter() - r0 < 0.1:
            run(tens)
            torch.cuda.synchronize()
        ms, wall = timed(lambda: run(tens), steps, 5, group=10 if tiny else 1)
        flops = sum(2.0 * N * K * C * H * H * 9 for (N, C, K, H) in layers)
        res = {"ms": round(ms, 4), "ms_wall_mean": round(wall, 4), "steps": steps,
               "effective_tflops": round(flops / (ms * 1e-3) / 1e12, 2), "dtype": dtype, "layout": layout_name}
        per_layer, k_flops, k_ms = [], 0.0, 0.0
        for (N, C, K, H), t in zip(layers, tens):
            a = ops.pick_algo(layout, DT[dtype], N, C, K, H, H)
            st = staged_pass(lambda: run([t]), 10)
            r = kernel_roofline(layout_name, dtype, a, N, C, K, H, st["gemm"][0] / 10)
            k_flops += r["flops"]
            k_ms += r["kernel_ms"]
            if many:
                lms, _ = timed(lambda: run([t]), 10, 2)
                per_layer.append({"C": C, "K": K, "H": H, "ms": round(lms, 4),
                                  "input_ms": round(st["input"][0] / 10, 4), **{k: r[k] for k in (
                                      "algo", "kernel_ms", "flop_per_byte", "achieved_tflops", "attainable_tflops",
                                      "frac_of_attainable", "bound")}})
            else:
                res.update(algo=r["algo"], kernel=r["kernel"], kernel_ms=r["kernel_ms"], frac=r["frac_mfma"],
                           attainable_tflops=r["attainable_tflops"], frac_of_attainable=r["frac_of_attainable"],
                           bound=r["bound"])
        if many:
            ach = k_flops / (k_ms * 1e-3) / 1e12
            res.update(kernel="per-layer choice", kernel_ms=round(k_ms, 4), frac=round(ach / MFMA_PEAK_TFLOPS[dtype], 4),
                       bound="per layer", layers=per_layer)
        del tens
        torch.cuda.empty_cache()
        return res

    def published_sweep():
        """The one measurement the reference commits (layoutTest/NHWC/result.num:1, made by layoutTest/NHWC/test.sh:3-8
        with convModule_NHWC_padding.cu:84-99): wrapedConv_NHWC at H = W = 22, C = K = 128, pad 1, fp32, N = 1 .. 128, the
        mean of 10 calls that each transform the filters and end in a device synchronisation -- on a GPU it does not name.
        Timed here the same way (`us_sync_each_call`), and back to back on the stream (`us_back_to_back`, median)."""
        ref_us = [51.939201, 53.334396, 83.395195, 107.584000, 180.300797, 320.105621, 645.052795, 1236.102295]
        Ns, sync_us, b2b_us, algos = [1, 2, 4, 8, 16, 32, 64, 128], [], [], []
        for N in Ns:
            (x, w, y), = device_tensors([(N, 128, 128, 22)], LAYOUT["NHWC"], "f32", 0x22)

            def call():
                ops.conv(x, w, 1, LAYOUT["NHWC"], out=y)
            r0 = time.perf_counter()
            while time.perf_counter() - r0 < 0.05:
                call()
                torch.cuda.synchronize()
            best = []
            for _ in range(5):                     # five times the reference's 10-call loop; the median loop counts
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(10):
                    call()
                    torch.cuda.synchronize()
                e1.record()
                torch.cuda.synchronize()
                best.append(e0.elapsed_time(e1) * 100.0)
            sync_us.append(round(statistics.median(best), 2))
            ms, _ = timed(call, 100, 10, group=10)
            b2b_us.append(round(ms * 1e3, 2))
            algos.append(ops.ALGO_NAMES[ops.pick_algo(LAYOUT["NHWC"], DT["f32"], N, 128, 128, 22, 22)])
        return {"what": "wrapedConv_NHWC fp32, H=W=22, C=K=128, pad 1, filter transform in every call", "N": Ns,
                "unit": "us per call", "us_sync_each_call": sync_us, "us_back_to_back": b2b_us, "algo": algos,
                "reference_us": [round(v, 2) for v in ref_us], "reference_hardware": "an NVIDIA GPU the reference does not name",
                "reference_source": "layoutTest/NHWC/result.num:1",
                "reference_over_this": [round(r / v, 2) for r, v in zip(ref_us, sync_us)]}

    layers = layers_of(args.workload)
    multi = len(layers) > 1
    layout, tdt, dt, algo = LAYOUT[args.layout], TDT[args.dtype], DT[args.dtype], ALGO[args.algo]
    es = 4 if args.dtype == "f32" else 2

    stack = None
    if args.workload == "vgg16_stack":
        if args.algo in ("staged_f4", "direct"):
            print("bench.py: the stack driver takes auto (which prepares F(4x4) and direct-path filters per layer where "
                  "it will run them), staged, epilogue or fused as a layer's algorithm", file=sys.stderr)
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

    # ---- timed region: exactly K steps after W warm-up steps ----------------------------
    ms_per_step, ms_wall = timed(step, args.steps, args.warmup)
    direct_flops = sum(2.0 * N * K * C * H * H * 9 for (N, C, K, H) in layers)
    value = direct_flops / (ms_per_step * 1e-3) / 1e12

    # ---- the same K steps again, the library bracketing every stage with HIP events --------
    st = staged_pass(step, args.steps)

    per_step = {k: (v[0] / args.steps) for k, v in st.items()}        # ms per step, summed over layers
    gemm_flops = alg_in = alg_out = alg_flt = 0.0
    resolved = []
    for (N, C, K, H) in layers:
        a = ops.pick_algo(layout, dt, N, C, K, H, H) if algo == ops.ALGO_AUTO else algo
        f4 = a in (ops.ALGO_STAGED_F4, ops.ALGO_EPILOGUE_F4)
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
    algo_label = resolved[0] if len(set(resolved)) == 1 else "mixed"
    traffic, traffic_source = MEASURED_TRAFFIC.get((args.workload, args.layout, args.dtype, algo_label), (None, None))
    roofline = {"bound": "mfma", "kernel": KERNEL_OF.get(algo_label, "per-layer choice"),
                "achieved": round(achieved, 2), "peak": peak, "unit": "TFLOP/s",
                "frac": round(achieved / peak, 4), "time_source": "HIP events the library records around the kernel on its launch stream",
                "traffic": traffic, "traffic_source": traffic_source,
                "flops_per_launch": gemm_flops if not multi else None}

    N0, C0, K0, H0 = layers[0]
    if not multi:
        # the dominant kernel's algorithmic bytes, its arithmetic intensity, and what the two roofs allow together
        r = kernel_roofline(args.layout, args.dtype, ops.pick_algo(layout, dt, N0, C0, K0, H0, H0)
                            if algo == ops.ALGO_AUTO else algo, N0, C0, K0, H0, gemm_ms)
        roofline.update(algorithmic_bytes=r["algorithmic_bytes"], flop_per_byte=r["flop_per_byte"],
                        attainable=r["attainable_tflops"], frac_of_attainable=r["frac_of_attainable"],
                        frac_hbm=round(r["GBps"] / HBM_PEAK_GBS, 3))
        if r["bound"] == "hbm":
            # the memory roof is the lower one for this kernel and type: it is the bound that is reported
            roofline.update(bound="hbm", achieved=r["GBps"], peak=HBM_PEAK_GBS, unit="GB/s",
                            frac=round(r["GBps"] / HBM_PEAK_GBS, 4), mfma_achieved=round(achieved, 2),
                            mfma_frac=round(achieved / peak, 4))
    out = {
        "metric": "effective TFLOP/s (direct-conv FLOPs), VGG-16 3x3 layer, N=32",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "ms_per_step_wall_mean": round(ms_wall, 4),
        "value_wall_mean": round(direct_flops / (ms_wall * 1e-3) / 1e12, 2),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": args.workload, "layers": len(layers), "N": N0, "C": C0, "K": K0, "H": H0, "W": H0,
                   "pad": 1, "layout": args.layout, "algo": args.algo, "resolved_algo": resolved,
                   "winograd": "F(4x4,3x3)" if algo_label in ("staged_f4", "epilogue_f4") else "F(2x2,3x3)",
                   "filter_transform_in_step": stack is None, "relu": multi,
                   "bias_and_pooling_in_step": stack is not None, "hip_graph": args.graph},
        "roofline": roofline,
        "stages": stages,
    }

    # ---- the same K steps with the filter bank transformed beforehand (filter transform excluded) ----
    if not multi and stack is None and resolved[0] in ("staged", "epilogue", "fused", "staged_f4", "epilogue_f4"):
        x0, w0, y0 = tensors[0]
        U0 = ops.f4_filter_transform(w0, layout) if resolved[0] in ("staged_f4", "epilogue_f4") else ops.filter_transform(w0, layout)
        a0 = {"staged": ops.ALGO_STAGED, "epilogue": ops.ALGO_EPILOGUE, "fused": ops.ALGO_FUSED,
              "staged_f4": ops.ALGO_STAGED_F4, "epilogue_f4": ops.ALGO_EPILOGUE_F4}[resolved[0]]
        out["ms_per_step_filters_prepared"] = round(
            timed(lambda: ops.conv_prepared(x0, U0, K0, 1, layout, algo=a0, out=y0), args.steps, args.warmup)[0], 4)

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
                ms, _ = timed(lambda: ops.layout_transform(a, la, lb), 100, 3, group=20)
                gbs = 2.0 * x0.numel() * es / (ms * 1e-3) / 1e9
                perms[f"{names[la]}->{names[lb]}"] = {"ms": round(ms, 4), "GBps": round(gbs, 1),
                                                      "frac_hbm": round(gbs / HBM_PEAK_GBS, 3)}
            del x1
        out["layout_transforms"] = perms

    # ---- the other benchmark configurations (default run only) ----------------------------------
    default_run = (args.workload == "vgg16_conv3_N32_C256_K256_H56" and args.layout == "NCHW" and args.dtype == "f32"
                   and args.algo == "auto")
    if default_run and not args.no_other_configs:
        del tensors
        torch.cuda.empty_cache()
        out["configs"] = {name: other_config(wl, dty, lay) for (name, wl, dty, lay) in OTHER_CONFIGS}
        out["configs"]["reference_published_sweep"] = published_sweep()

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
    # the last key of the line (a record that keeps only the line's tail still holds every configuration):
    # name -> [ms, effective TFLOP/s, AUTO's pipeline, dominant kernel's fraction of min(MFMA peak, flop/byte x 8 TB/s)]
    if "configs" in out:
        out["configs_summary"] = {name: [c["ms"], c["effective_tflops"], c.get("algo", "per layer"),
                                         c.get("frac_of_attainable", c.get("frac"))]
                                  for name, c in out["configs"].items() if "ms" in c}
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
