#!/usr/bin/env python3
"""Benchmark: int8 images/sec of the MobileNetV1-1.0-224-style network at batch 64 on one MI355X.

A step is one forward pass of the whole network over one batch that is already resident in HBM (every layer
runs on the device through the C ABI; the pass is replayed as one HIP graph).  Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 64] [--net mobilenet_v1|resnet50]
                  [--weights per_channel_s8|per_tensor_u8] [--no-cpu-baseline] [--layers]

The headline workload is the default: per-channel QSymmS8 weights.  --weights per_tensor_u8 runs the same network with
QAsymmU8 weights that have one scale and a zero point per layer, and says so in config.workload.

Extra objects in the line:
  roofline      the kernel with the largest share of the step (HIP-event timed on the launch stream)
  groups        conv/FC ops vs the int8 MFMA peak and depthwise bytes vs the HBM peak over the whole net
  cpu_baseline  the reference's own CpuRef code (oracle/_ref, kind "reference") or the C restatement
                (kind "port"), one thread, on a bounded sample of the same workload
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

INT8_MFMA_PEAK_OPS = 5.0e15      # MI355X dense int8, ops/s
HBM_PEAK_BYTES = 8.0e12          # MI355X HBM3E, B/s
RIDGE_OPS_PER_BYTE = INT8_MFMA_PEAK_OPS / HBM_PEAK_BYTES

# HBM bytes per launch (read + written) of each MobileNetV1 layer, keyed by the images one launch covers (32 = one of
# the two lanes of the default run), from two rocprofv3 --pmc passes (FETCH_SIZE, then WRITE_SIZE) over
# `python3 bench.py --profile-pass --no-graph` (batch-64 entries: `--lanes 1`), each scaled by what the same counter
# reads for the 64 MiB calibration copy of that pass (FETCH_SIZE counts 2 KiB units on this device: factor 1.999;
# WRITE_SIZE 1 KiB units: factor 1.000).  Summary: profiles/mobilenet_v1_b64_hbm_traffic.md.
MEASURED_HBM_TRAFFIC = {
    ("mobilenet_v1_1.0_224", 32): {
        "stem": 21485289,
        "dw1": 25858383,
        "pw1": 38751390,
        "dw2": 32236845,
        "pw2": 19656450,
        "dw3": 25886017,
        "pw3": 26132677,
        "dw4": 16206570,
        "pw4": 10235764,
        "dw5": 13085401,
        "pw5": 13540596,
        "dw6": 8216572,
        "pw6": 6180643,
        "dw7": 6736907,
        "pw7": 8934584,
        "dw8": 6733324,
        "pw8": 8931769,
        "dw9": 6733708,
        "pw9": 8932281,
        "dw10": 6734988,
        "pw10": 8931641,
        "dw11": 6732557,
        "pw11": 8932537,
        "dw12": 4223300,
        "pw12": 7106219,
        "dw13": 3586967,
        "pw13": 12327782,
        "avgpool": 1687743,
        "logits": 1453028,
        "softmax": 127440
    },
    ("mobilenet_v1_1.0_224", 64): {
        "dw1": 51482293,
        "pw1": 77282791,
        "dw2": 64298192,
        "pw2": 38912815,
        "dw3": 51513126,
        "pw3": 51807254,
        "dw4": 32217414,
        "pw4": 19858707,
        "dw5": 25869979,
        "pw5": 26564936,
        "dw6": 16205108,
        "pw6": 10982215,
        "dw7": 13107001,
        "pw7": 15305224,
        "dw8": 13106106,
        "pw8": 15305736,
        "dw9": 13104059,
        "pw9": 15306376,
        "dw10": 13104187,
        "pw10": 15305608,
        "dw11": 13104827,
        "pw11": 15306120,
        "dw12": 8241622,
        "pw12": 9543656,
        "dw13": 6807456,
        "pw13": 15567723,
        "softmax": 194497
    },
}


def layer_work(net, l, batch):
    """(kind, algorithmic work per launch): conv/fc -> ops = 2*MACs; others -> bytes, each tensor once."""
    if l.op in ("conv", "fc"):
        return "mfma", 2.0 * l.macs_per_image * batch
    if l.op == "dwpw":
        # fused depthwise + pointwise: the tensor between them never exists, so the unit's algorithmic bytes are its
        # input, its output and both layers' constants; priced against HBM like the depthwise layer it absorbs
        dw, pw = l.parts
        nbytes = (net.tensors[dw.inputs[0]].num_elements + net.tensors[pw.output].num_elements) * batch
        for part in (dw, pw):
            nbytes += part.weights.info.num_elements + 8 * net.tensors[part.output].shape[-1]
        return "hbm", float(nbytes)
    nbytes = sum(net.tensors[i].num_elements for i in l.inputs) + net.tensors[l.output].num_elements
    nbytes *= batch
    if l.weights is not None:
        co = net.tensors[l.output].shape[-1]
        nbytes += l.weights.info.num_elements + 8 * co     # + bias 4 B + per-channel scale 4 B
    return "hbm", float(nbytes)


def algorithmic_bytes(net, l, batch):
    """input(s) + output + weights + 8 B per output channel (bias, scale), each once, 1 B per 8-bit element."""
    n = (sum(net.tensors[i].num_elements for i in l.inputs) + net.tensors[l.output].num_elements) * batch
    if getattr(l, "weights", None) is not None:
        n += l.weights.info.num_elements + 8 * net.tensors[l.output].shape[-1]
    return n


def cpu_baseline(net, seconds_budget=25.0):
    from oracle import cpuref, netref
    from armnn_amd import nets
    kind = "reference" if cpuref.have("reference") else "port"
    if kind == "port" and not cpuref.have("port"):
        cpuref.build(reference=False)
    orc = cpuref.Oracle(kind)
    os.environ["OMP_NUM_THREADS"] = "1"
    images, elapsed = 0, 0.0
    while True:
        x = nets.synthetic_input(net, 1, seed=100 + images)
        t0 = time.perf_counter()
        netref.run_network(orc, net, x, fast=False)      # literal single-thread loop nest, as CpuRef runs it
        elapsed += time.perf_counter() - t0
        images += 1
        if elapsed * (images + 1) / images > seconds_budget or images >= 8:
            break
    return {"value": images / elapsed, "unit": "images/sec", "cores": 1, "kind": kind,
            "sample": f"{images} image(s) of the same network at batch 1, {elapsed:.1f} s, 1 thread of {os.cpu_count()}"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--net", default="mobilenet_v1", choices=["mobilenet_v1", "resnet50"])
    ap.add_argument("--weights", default="per_channel_s8", choices=["per_channel_s8", "per_tensor_u8"],
                    help="mobilenet_v1 only: per_tensor_u8 gives every layer QAsymmU8 weights with one scale and a zero point "
                         "(the quantization of older uint8 models) instead of the headline workload's per-channel QSymmS8")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--fuse", action="store_true",
                    help="run depthwise + pointwise pairs as one kernel (same bytes; slower than two launches at present)")
    ap.add_argument("--lanes", type=int, default=2,
                    help="split the batch into this many slices, each running the network on a stream of its own")
    ap.add_argument("--layers", action="store_true", help="print the per-layer table to stderr")
    ap.add_argument("--profile-pass", action="store_true",
                    help="for rocprofv3 --pmc: one 64 MiB calibration copy (1 B read + 1 B written per element), then ONE "
                         "eager forward pass, one kernel per layer in network order; prints the dispatch order as JSON")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus N with N > 1 is not supported "
              "(the path shards by batch with no exchange step: one process per GPU would run the same plans on its slice).", file=sys.stderr)
        return 2

    from armnn_amd import nets, shim
    from armnn_amd.executor import DeviceNetwork

    net = nets.mobilenet_v1(weights=args.weights) if args.net == "mobilenet_v1" else nets.resnet50()
    batch = args.batch
    dn = DeviceNetwork(net, batch, use_graph=not args.no_graph, fuse=args.fuse, lanes=args.lanes)
    dn.upload_input(nets.synthetic_input(net, batch))
    dev = dn.dev

    if args.profile_pass:
        import ctypes as C
        n = 64 << 20
        a, b = shim.DeviceBuffer(n), shim.DeviceBuffer(n)
        q = shim.Quant(0, 1.0, 0)
        shim._chk(dn.lib.mi355x_fill_u8(a.ptr, 1, n, dn.stream))
        dev.stream_sync(dn.stream)
        shim._chk(dn.lib.mi355x_activation_run(n, C.byref(q), C.byref(q), shim.ACT_BOUNDED_RELU, 1000.0, -1000.0, a.ptr, b.ptr, dn.stream))
        for _, fn in dn.steps:
            fn(dn.stream, 0, args.lanes)                 # lane 0's launch of every layer, as the timed region launches it
        dev.stream_sync(dn.stream)
        print(json.dumps({"dispatch_order": ["fill (setup)", f"calibration copy {n} B in + {n} B out"] + [l.name for l, _ in dn.steps],
                          "batch": batch, "launch_batch": batch // args.lanes, "net": net.name}))
        dn.close()
        return 0

    for _ in range(args.warmup):
        dn.enqueue()
    dev.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        dn.enqueue()
    dev.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    images_per_s = batch * args.steps / (t1 - t0)

    # ---- per-kernel timing on the launch stream, for the roofline object ------------------------------------
    # (one launch = one layer over one lane's slice of the batch; in the timed region `lanes` such launches of a layer
    # run side by side on their own streams)
    launch_batch = batch // args.lanes
    per_layer = dn.time_layers(iters=20, warmup=3)
    rows = []
    for l, ms in per_layer:
        kind, work = layer_work(net, l, launch_batch)
        peak = INT8_MFMA_PEAK_OPS if kind == "mfma" else HBM_PEAK_BYTES
        row = {"layer": l.name, "op": l.op, "ms": ms, "bound": kind, "work": work, "frac": work / (ms * 1e-3) / peak}
        if kind == "mfma":
            # the roof that binds a conv / FC layer depends on its arithmetic intensity: below the ridge
            # (peak ops / peak bytes = 625 ops/B) the HBM roof is the lower one
            nbytes = float(algorithmic_bytes(net, l, launch_batch))
            row["bytes"] = nbytes
            row["binding"] = "mfma" if work / nbytes >= RIDGE_OPS_PER_BYTE else "hbm"
        else:
            row["bytes"] = work
            row["binding"] = "hbm"
        rows.append(row)
    total_ms = sum(r["ms"] for r in rows)
    dom = max(rows, key=lambda r: r["ms"])
    if args.layers:
        for r in rows:
            hbm = r["bytes"] / (r["ms"] * 1e-3) / HBM_PEAK_BYTES
            print(f"{r['layer']:>10s} {r['op']:>9s} {r['ms']*1e3:9.1f} us  {r['bound']:>4s} {100*r['frac']:6.2f}% of peak"
                  f"   binding roof {r['binding']:>4s}, {100*hbm:5.1f}% of HBM peak on algorithmic bytes", file=sys.stderr)
        print(f"launches of {launch_batch} images; sum of one lane's launches {total_ms:.3f} ms; step of {args.lanes} lane(s) "
              f"{ms_per_step:.3f} ms", file=sys.stderr)
    if dom["binding"] == "mfma":
        roof = {"bound": "mfma", "achieved": dom["work"] / (dom["ms"] * 1e-3) / 1e12, "peak": INT8_MFMA_PEAK_OPS / 1e12,
                "unit": "TOP/s"}
    else:
        roof = {"bound": "hbm", "achieved": dom["bytes"] / (dom["ms"] * 1e-3) / 1e9, "peak": HBM_PEAK_BYTES / 1e9,
                "unit": "GB/s"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    roof["traffic"] = MEASURED_HBM_TRAFFIC.get((net.name, launch_batch), {}).get(dom["layer"])
    roof["kernel"] = (f"{dom['layer']} ({dom['op']}), one launch over {launch_batch} images: {dom['ms']*1e3:.1f} us of "
                      f"{total_ms*1e3:.1f} us for all layers")

    def group(ops, peak):
        sel = [r for r in rows if r["op"] in ops]
        t = sum(r["ms"] for r in sel) * 1e-3
        w = sum(r["work"] for r in sel)
        return {"ms": t * 1e3, "achieved": w / t, "frac": w / t / peak} if t > 0 else None

    g_conv = group(("conv", "fc"), INT8_MFMA_PEAK_OPS)
    g_dw = group(("depthwise", "dwpw"), HBM_PEAK_BYTES)
    groups = {
        "conv_fc": {"ms": g_conv["ms"], "TOPS": g_conv["achieved"] / 1e12, "frac_of_int8_mfma_peak": g_conv["frac"]},
    }
    if g_dw:
        groups["depthwise"] = {"ms": g_dw["ms"], "GBps": g_dw["achieved"] / 1e9, "frac_of_hbm_peak": g_dw["frac"]}

    line = {
        "metric": "int8 images/sec MobileNetV1 b64 @1 GPU" if args.net == "mobilenet_v1" else f"int8 images/sec {args.net} b{batch} @1 GPU",
        "value": images_per_s, "unit": "images/sec", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": f"{net.name} int8 (QAsymm activations, {'per-channel QSymmS8' if args.weights == 'per_channel_s8' or args.net != 'mobilenet_v1' else 'per-tensor QAsymmU8'} weights), batch {batch}, "
                               f"random-init, whole forward pass incl. avgpool/FC/softmax, input resident in HBM",
                   "batch": batch, "graph_replay": not args.no_graph, "fused_depthwise_pointwise": args.fuse, "lanes": args.lanes,
                   "total_TOPS": 2.0 * net.macs_per_image() * batch / (ms_per_step * 1e-3) / 1e12},
        "roofline": roof, "groups": groups,
    }
    # what the device itself delivers on register-only MFMA chains and on a plain copy, next to the published peaks
    from armnn_amd import peaks
    line["measured_peaks"] = peaks.measure()
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(net)
    dn.close()
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
