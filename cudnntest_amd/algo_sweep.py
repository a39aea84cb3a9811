"""Times every pipeline by name against the automatic choice over a grid of layer shapes, through the C ABI.

    python3 -m cudnntest_amd.algo_sweep --dtype f32 --layout NCHW [--dst NHWC] [--pool] [--quick]

One line per shape (microseconds, median of event-timed calls issued one after the other) and a summary: the sum of
the automatic choice's times, the sum of the fastest pipeline's, and the geometric mean of their ratio.  The rules
in resolve_auto (csrc/wino_api.hip) were fitted to these grids; a shape family of your own can be checked the same
way by editing GRIDS.  Needs a GPU; the library must be built (python3 -c "import __graft_entry__ as g; g.build()").
"""
import argparse
import itertools
import math
import statistics

import torch

from . import _lib, ops

ALGOS = {"staged": ops.ALGO_STAGED, "epilogue": ops.ALGO_EPILOGUE, "fused": ops.ALGO_FUSED, "f4": ops.ALGO_STAGED_F4,
         "direct": ops.ALGO_DIRECT}
# (channels, filters, (batch, image side)) per element type; the 2-byte grid stays at 28 x 28 and above, where the
# direct kernels are offered, and leaves F(4x4) out (its 2-byte rounding is not what the automatic choice may pick)
GRIDS = {
    "f32": ([48, 64, 96, 128, 192, 256, 384, 512], [16, 32, 64, 96, 128, 256],
            [(4, 56), (16, 56), (32, 56), (8, 112), (32, 28), (64, 14), (2, 160), (1, 112), (8, 40)]),
    "bf16": ([8, 16, 32, 64, 96, 128, 192, 256, 384, 512], [16, 32, 64, 96, 128, 256],
             [(1, 56), (4, 56), (16, 56), (32, 56), (2, 112), (8, 112), (1, 224), (4, 80), (16, 80), (32, 40), (8, 48),
              (32, 28)]),
}
GRIDS["f16"] = GRIDS["bf16"]
TORCH = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}
LAYOUTS = {"NCHW": ops.NCHW, "NHWC": ops.NHWC, "CHWN": ops.CHWN}


def timed(call, steps, warm=3):
    for _ in range(warm):
        call()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    ev[0].record()
    for i in range(steps):
        call()
        ev[i + 1].record()
    torch.cuda.synchronize()
    return statistics.median(ev[i].elapsed_time(ev[i + 1]) for i in range(steps)) * 1e3


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--dtype", choices=sorted(GRIDS), default="f32")
    ap.add_argument("--layout", choices=sorted(LAYOUTS), default="NCHW")
    ap.add_argument("--dst", choices=sorted(LAYOUTS), default=None, help="layout of y (default: that of x)")
    ap.add_argument("--pool", action="store_true", help="bias, ReLU and 2x2 pooling in the output stage")
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--quick", action="store_true", help="every third shape of the grid")
    ap.add_argument("--max-gflop", type=float, default=250.0, help="skip larger layers")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("algo_sweep needs a GPU")
    lay, tdt = LAYOUTS[args.layout], TORCH[args.dtype]
    dst = LAYOUTS[args.dst or args.layout]
    Cs, Ks, NHs = GRIDS[args.dtype]
    shapes = [(N, C, K, H) for (N, H), C, K in itertools.product(NHs, Cs, Ks)
              if 2.0 * N * C * K * H * H * 9 <= args.max_gflop * 1e9 and N * max(C, K) * H * H * 4 <= 6e8]
    if args.quick:
        shapes = shapes[::3]
    log_sum, auto_sum, best_sum = 0.0, 0.0, 0.0
    for (N, C, K, H) in shapes:
        x = (torch.rand((N, C, H, H), device="cuda") * 2 - 1).to(tdt)
        w = (torch.randn((K, C, 3, 3), device="cuda") * 0.05).to(tdt)
        b = torch.randn(K, device="cuda").to(tdt) if args.pool else None
        if lay == ops.NHWC:
            x, w = x.permute(0, 2, 3, 1).contiguous(), w.permute(0, 2, 3, 1).contiguous()
        if lay == ops.CHWN:
            x, w = x.permute(1, 2, 3, 0).contiguous(), w.permute(1, 2, 3, 0).contiguous()
        kw = dict(relu=True, bias=b, pool=True) if args.pool else {}
        y = ops.conv(x, w, 1, lay, dst, **kw)
        times = {}
        for name, algo in ALGOS.items():
            if name == "f4" and args.dtype != "f32":
                continue
            try:
                ops.conv(x, w, 1, lay, dst, out=y, algo=algo, **kw)
            except _lib.WinoError:          # the pipeline is not built for this shape
                continue
            times[name] = timed(lambda: ops.conv(x, w, 1, lay, dst, out=y, algo=algo, **kw), args.steps)
        auto = timed(lambda: ops.conv(x, w, 1, lay, dst, out=y, **kw), args.steps)
        best = min(times, key=times.get)
        log_sum += math.log(auto / times[best])
        auto_sum += auto
        best_sum += times[best]
        print(f"N{N} C{C} K{K} H{H}: auto {auto:.1f} best {best} {times[best]:.1f} x{auto / times[best]:.2f} | "
              + " ".join(f"{k}={v:.1f}" for k, v in times.items()), flush=True)
    n = max(len(shapes), 1)
    print(f"{len(shapes)} shapes, {args.dtype} {args.layout}{' -> ' + args.dst if args.dst else ''}{' pooled' if args.pool else ''}: automatic choice {auto_sum / 1e3:.2f} ms in all, "
          f"fastest by name {best_sum / 1e3:.2f} ms, geometric mean of the ratio {math.exp(log_sum / n):.3f}")


if __name__ == "__main__":
    main()
