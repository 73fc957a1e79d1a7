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
  configs      the other BASELINE configs (1 at one image and as 256 replicas, 2 at batch 256, 4 at batch 64,
               5 at batch 512), each timed the same way in the same run: ms per step, images/s, int8 TOP/s, the
               kernel family that takes the most time with its fractions of both roofs, parity_checked
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
    "mbconv_s8_wave": 42770000.0,   # 7 launches (the stem convolution rides in the first block's launch)
    "mbconv_s8_group": 8491849.0,   # 10 launches
    "conv2d_s8": 7173205.0,         # head convolution with GlobalAveragePool, classifier
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
    if info["type"] in ("Concat", "Split") and info["bytes"] == 0:
        return "view"  # every piece is a channel slice of the wide tensor: nothing is launched
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


# The VALU floor of the fused inverted-residual kernels: every stage result is requantized on the vector ALU
# (shift, saturating convert, clamp, byte gather: 11 instructions per four values when a layer has a shift below
# 8), and a SIMD issues one vector instruction per 4 cycles.  1024 SIMDs x 2.4 GHz / 4 x 64 lanes x 4 / 11 values.
VALU_PEAK_GVALUES = 1024 * 2.4e9 / 4.0 * 64 * 4.0 / 11.0 / 1e9


def requantized_values(spec, module_name, kind):
    """Stage outputs of a fused block (per image): the values its launch requantizes on the vector ALU.  The
    module carries the name of its depthwise node; the project Conv behind it and, for a whole block, the Conv
    in front (looking through a clamp-only Clip on either side) are the other stages."""
    by_name = {n["name"]: n for n in spec.nodes}
    producer = {o: n for n in spec.nodes for o in n["outputs"]}
    readers = {}
    for n in spec.nodes:
        for i in n["inputs"]:
            readers.setdefault(i, []).append(n)
    dw = by_name.get(module_name)
    if dw is None:
        return 0

    def elements(node):
        r = 1
        for x in spec.shape(node["outputs"][0])[1:]:
            r *= int(x)
        return r

    total = elements(dw)
    nxt = readers.get(dw["outputs"][0], [None])[0]
    if nxt is not None and nxt["op_type"] == "Clip":
        nxt = readers.get(nxt["outputs"][0], [None])[0]
    if nxt is not None and nxt["op_type"] == "Conv":
        total += elements(nxt)
    if kind.count(">") == 2:
        prev = producer.get(dw["inputs"][0])
        if prev is not None and prev["op_type"] == "Clip":
            prev = producer.get(prev["inputs"][0])
        if prev is not None and prev["op_type"] == "Conv":
            total += elements(prev)
    return total


def measure(pkg, args, config, batch, steps, warmup, parity=True, layers=False):
    """One workload: K timed HIP-graph replays bracketed by synchronization, per-family HIP-event times from
    whole passes of the plan, then (outside every timed region) the comparison with the CPU oracle."""
    import numpy as np
    import torch
    spec = pkg.zoo.CONFIGS[config]()
    graph = pkg.model.Graph.from_spec(spec)
    mdl = pkg.model.Model(graph, batch, fuse_add=not args.no_fuse_add, fuse_gap=not args.no_fuse_gap)
    x = spec.make_input(np.random.default_rng(0xE5D10000 + config), batch)
    mdl.set_input(spec.inputs[0], x)  # resident in HBM from here on
    mdl.run()
    use_graph = (not args.no_graph) and mdl.enable_graph()
    for _ in range(warmup):
        mdl.run_async()
    mdl.synchronize()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        mdl.run_async()
    mdl.synchronize()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / steps
    out_np = {name: mdl.get_tensor(name, np.int16 if spec.dtype(name) == 5 else np.int8) for name in spec.outputs}
    checksum = int(sum(int(v.astype(np.int64).sum()) for v in out_np.values()))
    # per-kernel timing with HIP events on the model's stream (eager launches of the same plan)
    mdl.disable_graph()
    nodes = {n["name"]: n for n in spec.nodes}
    fam = {}
    for info in mdl.profile(repeats=args.profile_repeats):
        f = kernel_family(info, nodes)
        if layers:
            print("%-28s %-8s %-16s %9.2f us %8.1f GB/s %8.2f TOP/s" % (
                info["name"], info["type"], f, info["latency_us"], info["bytes"] / max(info["latency_us"], 1e-3) * 1e-3,
                2.0 * info["macs"] / max(info["latency_us"], 1e-3) * 1e-6), file=sys.stderr)
        d = fam.setdefault(f, {"us": 0.0, "macs": 0, "bytes": 0, "launches": 0, "values": 0})
        d["us"] += info["latency_us"]
        d["macs"] += info["macs"]
        d["bytes"] += info["bytes"]
        d["launches"] += 1
        if f.startswith("mbconv_s8"):
            d["values"] += requantized_values(spec, info["name"], info["type"].partition(":")[0]) * batch
    # the comparison with the oracle keeps the host busy and the GPU idle for about a second; it comes after the
    # per-kernel timing so that the kernels are timed at the clocks of the timed region
    parity_checked = check_against_oracle(spec, x, out_np) if parity else None
    modules = mdl.module_count()
    mdl.close()

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
        if d["values"]:
            gv = d["values"] / d["us"] * 1e-3
            kernels[f]["requantized_values_per_step"] = d["values"]
            kernels[f]["Gvalues_per_s"] = round(gv, 1)
            kernels[f]["valu_frac"] = round(gv / VALU_PEAK_GVALUES, 4)
    return {"spec": spec, "batch": batch, "ms_per_step": ms_per_step, "images_per_s": batch * steps / elapsed,
            "checksum": checksum, "parity_checked": parity_checked, "kernels": kernels, "modules": modules,
            "hip_graph": bool(use_graph), "int8_tops": 2.0 * spec.macs_per_image * batch / (ms_per_step * 1e-3) / 1e12}


def dominant_roofline(kernels):
    """The kernel family that takes the most time, against the roof that bounds it.  The fused block kernels
    keep their expanded activations on chip: neither HBM (a few percent of their time) nor the matrix pipe binds
    them but the vector ALU, which requantizes every stage's result; they are priced against that floor, with the
    fractions of both published roofs next to it."""
    dom = max(kernels, key=lambda k: kernels[k]["us_per_step"])
    kd = kernels[dom]
    if "valu_frac" in kd:
        roofline = {"kernel": dom, "bound": "valu", "achieved": kd["Gvalues_per_s"], "peak": round(VALU_PEAK_GVALUES, 1),
                    "unit": "G requantized values/s", "frac": kd["valu_frac"], "traffic": None,
                    "peak_note": "1024 SIMDs x 2.4 GHz / 4 cycles x 64 lanes x 4 values / 11 instructions"}
        per_launch = kd["requantized_values_per_step"] / kd["launches_per_step"]
    elif (dom == "conv2d_s8" or dom.startswith("mbconv_s8")) and kd["ops_per_byte"] > MACHINE_BALANCE:
        roofline = {"kernel": dom, "bound": "mfma", "achieved": kd["TOPs"], "peak": PEAK_INT8_TOPS,
                    "unit": "TOP/s", "frac": kd["mfma_frac"], "traffic": None}
        per_launch = kd["algorithmic_ops_per_step"] / kd["launches_per_step"]
    else:
        roofline = {"kernel": dom, "bound": "hbm", "achieved": kd["GBps"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                    "frac": kd["hbm_frac"], "traffic": None}
        per_launch = kd["algorithmic_bytes_per_step"] / kd["launches_per_step"]
    roofline["frac_hbm"] = kd["hbm_frac"]
    roofline["frac_mfma"] = kd["mfma_frac"]
    roofline["launches_per_step"] = kd["launches_per_step"]
    roofline["avg_launch_us"] = kd["avg_launch_us"]
    roofline["algorithmic_per_launch"] = per_launch
    roofline["algorithmic_bytes_per_launch"] = kd["algorithmic_bytes_per_step"] / kd["launches_per_step"]
    return roofline


# the other BASELINE configs reported next to the headline: (config, batch)
OTHER_CONFIGS = [(1, 1), (1, 256), (2, 256), (4, 64), (5, 512)]


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
    ap.add_argument("--no-configs", action="store_true", help="skip the other BASELINE configs (the `configs` object)")
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

    batch = args.batch
    m = measure(pkg, args, args.config, batch, args.steps, args.warmup, parity=not args.no_parity, layers=args.layers)
    spec, kernels = m["spec"], m["kernels"]
    roofline = dominant_roofline(kernels)
    if args.config == 3 and batch == 256:
        roofline["traffic"] = MEASURED_TRAFFIC_BYTES_PER_LAUNCH.get(roofline["kernel"])

    result = {
        "metric": ("images/sec + int8 TOPS (% roofline), MobileNetV2-224 int8, batch 256"
                   if args.config == 3 and batch == 256 else
                   "images/sec + int8 TOPS (%% roofline), %s, batch %d" % (spec.name, batch)),
        "value": round(m["images_per_s"], 1), "unit": "images/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(m["ms_per_step"], 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "s8", "data": "synthetic",
        "config": {"workload": "%s, batch %d (BASELINE config %d)" % (spec.name, batch, args.config),
                   "nodes": len(spec.nodes), "modules": m["modules"], "hip_graph": m["hip_graph"],
                   "macs_per_image": spec.macs_per_image, "round_mode": "half_up", "exponents": "per-channel"},
        "int8_tops": round(m["int8_tops"], 2),
        "int8_mfma_frac": round(m["int8_tops"] / PEAK_INT8_TOPS, 4),
        "output_checksum": m["checksum"],
        "parity_checked": m["parity_checked"],
        "roofline": roofline,
        "kernels": kernels,
    }
    bad_parity = m["parity_checked"] is False
    if not args.no_configs and args.config == 3 and batch == 256:
        # the other four BASELINE configs, same procedure, fewer steps; the CPU leg stays on the headline workload
        configs = {}
        for cfg, b in OTHER_CONFIGS:
            # (steps of config 1 take 15 and 50 us: many more of them, or the clock reads launch jitter and the
            # ramp of the GPU's clocks)
            k = args.steps * 5 if cfg == 1 else max(20, args.steps // 4)
            o = measure(pkg, args, cfg, b, k, max(5, args.warmup // 2) * (10 if cfg == 1 else 1), parity=not args.no_parity)
            r = dominant_roofline(o["kernels"])
            configs["config%d_batch%d" % (cfg, b)] = {
                "workload": "%s, batch %d" % (o["spec"].name, b), "ms_per_step": round(o["ms_per_step"], 4),
                "images_per_s": round(o["images_per_s"], 1), "int8_tops": round(o["int8_tops"], 2),
                "int8_mfma_frac": round(o["int8_tops"] / PEAK_INT8_TOPS, 4), "modules": o["modules"],
                "parity_checked": o["parity_checked"],
                "dominant_kernel": {"kernel": r["kernel"], "bound": r["bound"], "us_per_step": o["kernels"][r["kernel"]]["us_per_step"],
                                    "launches_per_step": r["launches_per_step"], "frac": r["frac"],
                                    "frac_hbm": r["frac_hbm"], "frac_mfma": r["frac_mfma"]},
                "kernel_us": {k: v["us_per_step"] for k, v in o["kernels"].items()},
            }
            bad_parity = bad_parity or o["parity_checked"] is False
        result["configs"] = configs
    if not args.no_cpu:
        threads = min(16, os.cpu_count() or 1)
        result["cpu_baseline"] = cpu_baseline(pkg, spec, threads)
    print(json.dumps(result))
    if bad_parity:
        sys.exit(3)


if __name__ == "__main__":
    main()
