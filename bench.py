#!/usr/bin/env python3
"""Headline benchmark: MobileNetV2-224 int8 (BASELINE config 3), batch 256, one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 256] [--config 3] [--no-cpu]

A step is one pass of the quantized operator path (dl::Model::run over the whole batch) with the
input batch already resident in HBM.  Prints ONE JSON line:
  value        images/s over the timed K steps (wall clock bracketed by device synchronization)
  int8_tops    2 * MACs of the Conv/Gemm layers per second, in TOP/s
  roofline     the kernel family that takes the most GPU time in a step: algorithmic bytes (or
               operations) of its launches divided by their HIP-event time, against MI355X's peak
  kernels      the same for every kernel family (conv/gemm on MFMA, depthwise, element-wise)
  parity_checked  true when every output of the timed batch equals the CPU oracle's bit for bit (checked
               after the timed region; the program exits with status 3 when it does not)
  cpu_baseline the CPU oracle (a port of the reference's portable C path) timed on this host's
               cores on a bounded sample of the same workload
Synthetic data: seeded uniform int8 images, random-init int8 weights with per-channel exponents.
"""
import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)

PEAK_HBM_GBS = 8000.0        # MI355X HBM3E, published
PEAK_INT8_TOPS = 5000.0      # MI355X dense int8 MFMA, published (5.0 POP/s)
MACHINE_BALANCE = PEAK_INT8_TOPS * 1e12 / (PEAK_HBM_GBS * 1e9)  # OP per byte

# HBM bytes per launch (average over the launches of a step) of the default workload, from two
# rocprofv3 counter runs of this program (FETCH_SIZE scaled by 2.0, WRITE_SIZE by 1.0: the factors a
# 256 MiB element-wise kernel of known traffic gave in the same runs).  Only valid for config 3 at
# batch 256; any other workload reports null.
MEASURED_TRAFFIC_BYTES_PER_LAUNCH = {
    "mbconv_s8_wave": 43233941.0,   # 7 launches (the stem convolution rides in the first block's launch)
    "mbconv_s8_group": 8492449.0,   # 10 launches
    "conv2d_s8": 7164469.0,         # head convolution with GlobalAveragePool, classifier
    "elementwise_s8": None,
}


def kernel_family(info, spec_nodes):
    """Map a module to the kernel that runs it."""
    node = spec_nodes.get(info["name"])
    kind, _, kernel = info["type"].partition(":")
    if kind == "Conv>DepthwiseConv>Conv":
        # expand + depthwise + project (+ Add) in one launch: the one-wavefront-per-tile kernel for the large
        # images, the workgroup-per-tile kernel for the small ones
        return "mbconv_s8_" + kernel if kernel in ("wave", "group") else "mbconv_s8"
    if kind == "DepthwiseConv>Conv":
        return "depthwise_s8"  # depthwise + project (+ Add) in one launch of the depthwise kernel
    if info["type"] in ("Gemm", "MatMul"):
        return "conv2d_s8"
    if info["type"] == "Conv":
        if node and node["attrs"].get("quant_type") == "S16":
            return "depthwise_s16" if node["attrs"].get("group", 1) != 1 else "conv2d_s16"
        return "depthwise_s8" if node and node["attrs"].get("group", 1) != 1 else "conv2d_s8"
    if info["type"] in ("Flatten", "Squeeze", "Reshape", "Unsqueeze"):
        return "view"
    return "elementwise_s8"


def cpu_baseline(pkg, spec, threads_all):
    """Time the oracle graph runner: single thread (the reference's execution model) and all cores."""
    import numpy as np
    import espdl_oracle as oracle
    import graph_runner
    rng = np.random.default_rng(0xC0FFEE)
    out = {}
    # calibrate on one image, single thread
    oracle.set_threads(1)
    x1 = spec.make_input(rng, 1)
    t0 = time.perf_counter()
    graph_runner.run(spec, {spec.inputs[0]: x1}, keep_all=False)
    t_one = time.perf_counter() - t0
    n1 = max(1, min(64, int(round(8.0 / max(t_one, 1e-3)))))
    x = spec.make_input(rng, n1)
    t0 = time.perf_counter()
    graph_runner.run(spec, {spec.inputs[0]: x}, keep_all=False)
    t1 = time.perf_counter() - t0
    out["single_thread_images_per_s"] = n1 / t1
    out["single_thread_sample"] = "%d images in %.2f s" % (n1, t1)
    # all cores: OpenMP over batch*rows inside every oracle call
    oracle.set_threads(threads_all)
    # size the sample from a short multi-thread pass so that the timed one takes about 15 s
    ncal = 4 * threads_all
    x = spec.make_input(rng, ncal)
    t0 = time.perf_counter()
    graph_runner.run(spec, {spec.inputs[0]: x}, keep_all=False)
    t_cal = time.perf_counter() - t0
    nall = max(threads_all, min(8192, int(round(15.0 * ncal / max(t_cal, 1e-3)))))
    nall -= nall % threads_all
    chunk = 256  # images per oracle call: bounds host memory (activations of every layer are kept per call)
    done, tall = 0, 0.0
    while done < nall:
        n = min(chunk, nall - done)
        x = spec.make_input(rng, n)
        t0 = time.perf_counter()
        graph_runner.run(spec, {spec.inputs[0]: x}, keep_all=False)
        tall += time.perf_counter() - t0
        done += n
    gmacs = spec.macs_per_image * nall / tall / 1e9
    return {
        "value": nall / tall, "unit": "images/s", "cores": threads_all, "kind": "port",
        "sample": "%d images of %s in %.2f s on %d threads (%.1f GMAC/s); 1 thread: %s = %.2f images/s"
                  % (nall, spec.name, tall, threads_all, gmacs, out["single_thread_sample"],
                     out["single_thread_images_per_s"]),
    }


def check_against_oracle(spec, x, got, chunk=32):
    """True when every graph output equals the oracle's, bit for bit."""
    import numpy as np
    import espdl_oracle as oracle
    import graph_runner
    oracle.set_threads(min(16, os.cpu_count() or 1))
    ok = True
    for i in range(0, x.shape[0], chunk):
        want = graph_runner.run(spec, {spec.inputs[0]: x[i:i + chunk]}, keep_all=False)
        for name in spec.outputs:
            g = got[name][i:i + chunk]
            if not np.array_equal(g.reshape(want[name].shape), want[name]):
                bad = int((g.reshape(want[name].shape) != want[name]).sum())
                print("bench.py: output %s of images %d..%d differs from the oracle in %d elements"
                      % (name, i, i + chunk - 1, bad), file=sys.stderr)
                ok = False
    return ok


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--batch", type=int, default=256)
    ap.add_argument("--config", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-parity", action="store_true", help="skip the comparison of the timed batch with the oracle")
    ap.add_argument("--no-graph", action="store_true", help="launch kernels eagerly instead of HIP-graph replay")
    ap.add_argument("--profile-repeats", type=int, default=5)
    ap.add_argument("--layers", action="store_true", help="print the per-module timing table to stderr")
    ap.add_argument("--no-fuse-gap", action="store_true",
                    help="run GlobalAveragePool as a module of its own instead of inside the 1x1 convolution before it")
    ap.add_argument("--no-fuse-add", action="store_true",
                    help="keep residual Adds as separate kernels instead of folding them into the conv before them")
    ap.add_argument("--copy-mib", type=int, default=0,
                    help="also run one plain device copy of this many MiB (a kernel of known traffic, the "
                         "yardstick for FETCH_SIZE / WRITE_SIZE counter runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported (images are independent, "
              "more GPUs would each take batch/N with a copy of the weights)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    pkg = importlib.import_module("esp-dl_amd")
    pkg.lib()  # fails loudly when the HIP library is missing

    if args.copy_mib > 0:
        src = torch.randint(-128, 128, (args.copy_mib << 20,), dtype=torch.int8, device="cuda")
        dst = torch.empty_like(src)
        torch.add(src, 1, out=dst)  # an element-wise kernel: reads and writes copy_mib MiB each
        torch.cuda.synchronize()
        del src, dst

    spec = pkg.zoo.CONFIGS[args.config]()
    batch = args.batch
    graph = pkg.model.Graph.from_spec(spec)
    mdl = pkg.model.Model(graph, batch, fuse_add=not args.no_fuse_add, fuse_gap=not args.no_fuse_gap)
    x = spec.make_input(np.random.default_rng(0xE5D10003), batch)
    mdl.set_input(spec.inputs[0], x)  # resident in HBM from here on
    mdl.run()
    use_graph = (not args.no_graph) and mdl.enable_graph()

    for _ in range(args.warmup):
        mdl.run_async()
    mdl.synchronize()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        mdl.run_async()
    mdl.synchronize()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    images_per_s = batch * args.steps / elapsed
    out_np = {name: mdl.get_tensor(name, np.int16 if spec.dtype(name) == 5 else np.int8) for name in spec.outputs}
    checksum = int(sum(int(v.astype(np.int64).sum()) for v in out_np.values()))
    # per-kernel timing with HIP events on the model's stream (eager launches of the same plan)
    mdl.disable_graph()
    nodes = {n["name"]: n for n in spec.nodes}
    fam = {}
    for info in mdl.profile(repeats=args.profile_repeats):
        f = kernel_family(info, nodes)
        if args.layers:
            print("%-28s %-8s %-16s %9.2f us %8.1f GB/s %8.2f TOP/s" % (
                info["name"], info["type"], f, info["latency_us"], info["bytes"] / max(info["latency_us"], 1e-3) * 1e-3,
                2.0 * info["macs"] / max(info["latency_us"], 1e-3) * 1e-6), file=sys.stderr)
        d = fam.setdefault(f, {"us": 0.0, "macs": 0, "bytes": 0, "launches": 0})
        d["us"] += info["latency_us"]
        d["macs"] += info["macs"]
        d["bytes"] += info["bytes"]
        d["launches"] += 1
    # the comparison with the oracle keeps the host busy and the GPU idle for about a second; it comes after the
    # per-kernel timing so that the kernels are timed at the clocks of the timed region
    parity_checked = None
    if not args.no_parity:
        # outside the timed region: every output of the batch that was just timed (the result of the last
        # timed step) against the CPU oracle on the same seeded input, in chunks of images
        parity_checked = check_against_oracle(spec, x, out_np)

    kernels = {}
    for f, d in fam.items():
        if f == "view" or d["us"] <= 0:
            continue
        gbs = d["bytes"] / d["us"] * 1e-3
        tops = 2.0 * d["macs"] / d["us"] * 1e-6
        ai = 2.0 * d["macs"] / max(1, d["bytes"])
        kernels[f] = {"launches_per_step": d["launches"], "us_per_step": round(d["us"], 2),
                      "avg_launch_us": round(d["us"] / d["launches"], 3),
                      "algorithmic_bytes_per_step": d["bytes"], "algorithmic_ops_per_step": 2 * d["macs"],
                      "GBps": round(gbs, 1), "hbm_frac": round(gbs / PEAK_HBM_GBS, 4),
                      "TOPs": round(tops, 2), "mfma_frac": round(tops / PEAK_INT8_TOPS, 4),
                      "ops_per_byte": round(ai, 1)}
    dom = max(kernels, key=lambda k: kernels[k]["us_per_step"])
    kd = kernels[dom]
    # time per family comes from whole passes in plan order, so the family times add up to a step
    if (dom == "conv2d_s8" or dom.startswith("mbconv_s8")) and kd["ops_per_byte"] > MACHINE_BALANCE:
        roofline = {"kernel": dom, "bound": "mfma", "achieved": kd["TOPs"], "peak": PEAK_INT8_TOPS,
                    "unit": "TOP/s", "frac": kd["mfma_frac"], "traffic": None}
    else:
        roofline = {"kernel": dom, "bound": "hbm", "achieved": kd["GBps"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                    "frac": kd["hbm_frac"], "traffic": None}
    if args.config == 3 and batch == 256:
        roofline["traffic"] = MEASURED_TRAFFIC_BYTES_PER_LAUNCH.get(dom)
    roofline["frac_hbm"] = kd["hbm_frac"]
    roofline["frac_mfma"] = kd["mfma_frac"]
    roofline["launches_per_step"] = kd["launches_per_step"]
    roofline["avg_launch_us"] = kd["avg_launch_us"]
    roofline["algorithmic_per_launch"] = (kd["algorithmic_ops_per_step"] if roofline["bound"] == "mfma"
                                          else kd["algorithmic_bytes_per_step"]) / kd["launches_per_step"]

    conv_macs = spec.macs_per_image * batch
    result = {
        "metric": ("images/sec + int8 TOPS (% roofline), MobileNetV2-224 int8, batch 256"
                   if args.config == 3 and batch == 256 else
                   "images/sec + int8 TOPS (%% roofline), %s, batch %d" % (spec.name, batch)),
        "value": round(images_per_s, 1), "unit": "images/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "s8", "data": "synthetic",
        "config": {"workload": "%s, batch %d (BASELINE config %d)" % (spec.name, batch, args.config),
                   "nodes": len(spec.nodes), "modules": mdl.module_count(), "hip_graph": bool(use_graph),
                   "macs_per_image": spec.macs_per_image, "round_mode": "half_up", "exponents": "per-channel"},
        "int8_tops": round(2.0 * conv_macs / (ms_per_step * 1e-3) / 1e12, 2),
        "int8_mfma_frac": round(2.0 * conv_macs / (ms_per_step * 1e-3) / 1e12 / PEAK_INT8_TOPS, 4),
        "output_checksum": checksum,
        "parity_checked": parity_checked,
        "roofline": roofline,
        "kernels": kernels,
    }
    if not args.no_cpu:
        threads = min(16, os.cpu_count() or 1)
        result["cpu_baseline"] = cpu_baseline(pkg, spec, threads)
    mdl.close()
    print(json.dumps(result))
    if parity_checked is False:
        sys.exit(3)


if __name__ == "__main__":
    main()
