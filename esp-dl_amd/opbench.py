#!/usr/bin/env python3
"""Achieved HBM bandwidth of the bandwidth-bound operators, one MI355X.

    python esp-dl_amd/opbench.py [--mib 256] [--reps 20] [--only maxpool]

Every operator runs through the C ABI on tensors of at least `--mib` MiB, timed with HIP events around `--reps`
back-to-back launches on the current stream; bandwidth = algorithmic bytes (every input and output byte once)
/ time, against the published 8 TB/s.  Prints one table line per operator.  Under
`rocprofv3 --kernel-trace --stats` the kernel names and durations of the same launches can be read next to it.
"""
import argparse
import importlib
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--mib", type=int, default=256)
    ap.add_argument("--reps", type=int, default=20)
    ap.add_argument("--only", default="", help="run only the operators whose line contains this text")
    args = ap.parse_args()
    import torch
    m = importlib.import_module("esp-dl_amd")
    m.lib()
    dev = "cuda"
    size = args.mib << 20

    def rand(shape):
        return torch.randint(-128, 128, shape, dtype=torch.int8, device=dev)

    def timed(name, fn, nbytes):
        if args.only.lower() not in name.lower():
            return
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / args.reps
        gbs = nbytes / us * 1e-3
        print("%-44s %9.1f MiB %10.2f us %9.1f GB/s   %.3f of HBM peak" % (name, nbytes / 2**20, us, gbs, gbs / PEAK_HBM_GBS),
              flush=True)

    # element-wise operators on a flat tensor viewed as [N, 64, 64, 64]
    n = max(1, size // (64 * 64 * 64))
    x = rand((n, 64, 64, 64))
    y = rand((n, 64, 64, 64))
    out = torch.empty_like(x)
    table = torch.arange(-128, 128, dtype=torch.int16, device=dev).flip(0).to(torch.int8)
    alpha = rand((64,))
    timed("LUT (espdl_hip_lut_s8)", lambda: m.lut_s8(x, table, out=out), 2 * x.numel())
    timed("Clip, equal exponents (espdl_hip_clip_s8)", lambda: m.clip_s8(x, 0, 96, out=out), 2 * x.numel())
    timed("Relu (espdl_hip_relu_s8)", lambda: m.relu_s8(x, out=out), 2 * x.numel())
    timed("PRelu, 64 channels (espdl_hip_prelu_s8)", lambda: m.prelu_s8(x, alpha, 6, out=out), 2 * x.numel())
    timed("RequantizeLinear e-5 -> e-7 (espdl_hip_requantize_s8)", lambda: m.requantize_s8(x, -5, -7, out=out), 2 * x.numel())
    timed("Add (espdl_hip_add_s8)", lambda: m.add_s8(x, y, out=out), 3 * x.numel())
    timed("Mul, shift 7 (espdl_hip_mul_s8)", lambda: m.mul_s8(x, y, 7, out=out), 3 * x.numel())
    del y

    # Concat / Split along channels: two halves of 64 channels <-> 128 channels
    cat = torch.empty((n, 64, 64, 128), dtype=torch.int8, device=dev)
    timed("Concat 64 + 64 channels (espdl_hip_concat)", lambda: m.concat([x, out], 3, out=cat), 2 * cat.numel())
    timed("Split 128 -> 64 + 64 channels (espdl_hip_split)", lambda: m.split(cat, 3, [64, 64]), 2 * cat.numel())
    del cat

    # MaxPool 5x5 stride 1 (SPPF), Resize nearest x2, on 80 x 80 x 128 images
    nb = max(1, size // (80 * 80 * 128))
    xi = rand((nb, 80, 80, 128))
    oi = torch.empty_like(xi)
    timed("MaxPool 5x5 s1 p2 (espdl_hip_max_pool)", lambda: m.max_pool(xi, (5, 5), (1, 1), (2, 2, 2, 2), out=oi), 2 * xi.numel())
    nr = max(1, nb // 4)
    xr = xi[:nr].contiguous()
    orr = torch.empty((nr, 160, 160, 128), dtype=torch.int8, device=dev)
    timed("Resize nearest x2 (espdl_hip_resize_nearest_s8)", lambda: m.resize_nearest_s8(xr, 2.0, 2.0, out=orr),
          xr.numel() + orr.numel())
    del xi, oi, xr, orr

    # depthwise 3x3 stride 1 on 56 x 56 x 144 (the depthwise stage of BASELINE config 2), on its own
    nd = max(1, size // (56 * 56 * 144))
    xd = rand((nd, 56, 56, 144))
    od = torch.empty_like(xd)
    f = rand((3, 3, 144))
    bias = torch.randint(-4096, 4096, (144,), dtype=torch.int32, device=dev)
    shift = torch.randint(8, 12, (144,), dtype=torch.int32, device=dev)
    timed("Depthwise 3x3 s1 p1, 144 channels (espdl_hip_conv2d)",
          lambda: m.conv2d(xd, f, bias, shift, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), depthwise=True, activation=m.capi.RELU, out=od),
          2 * xd.numel())
    # global average pool 7 x 7 x 1280 (MobileNetV2's head when it is not fused into the convolution)
    ng = max(1, size // (7 * 7 * 1280))
    xg = rand((ng, 7, 7, 1280))
    og = torch.empty((ng, 1, 1, 1280), dtype=torch.int8, device=dev)
    timed("GlobalAveragePool 7x7x1280 (espdl_hip_global_avg_pool_s8)", lambda: m.global_avg_pool_s8(xg, -4, -3, out=og),
          xg.numel() + og.numel())


if __name__ == "__main__":
    main()
