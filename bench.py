#!/usr/bin/env python3
"""Benchmark: int8 images/sec of the MobileNetV1-1.0-224-style network at batch 64 on one MI355X.

A step is one forward pass of the whole network over one batch that is already resident in HBM (every layer
runs on the device through the C ABI; the pass is replayed as one HIP graph).  Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 64] [--net mobilenet_v1|resnet50]
                  [--no-cpu-baseline] [--layers]

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
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--fuse", action="store_true",
                    help="run depthwise + pointwise pairs as one kernel (same bytes; slower than two launches at present)")
    ap.add_argument("--layers", action="store_true", help="print the per-layer table to stderr")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus N with N > 1 is not supported "
              "(the path shards by batch with no exchange step, see DESIGN.md).", file=sys.stderr)
        return 2

    from armnn_amd import nets, shim
    from armnn_amd.executor import DeviceNetwork

    net = nets.mobilenet_v1() if args.net == "mobilenet_v1" else nets.resnet50()
    batch = args.batch
    dn = DeviceNetwork(net, batch, use_graph=not args.no_graph, fuse=args.fuse)
    dn.upload_input(nets.synthetic_input(net, batch))
    dev = dn.dev

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
    per_layer = dn.time_layers(iters=20, warmup=3)
    rows = []
    for l, ms in per_layer:
        kind, work = layer_work(net, l, batch)
        peak = INT8_MFMA_PEAK_OPS if kind == "mfma" else HBM_PEAK_BYTES
        rows.append({"layer": l.name, "op": l.op, "ms": ms, "bound": kind, "work": work, "frac": work / (ms * 1e-3) / peak})
    total_ms = sum(r["ms"] for r in rows)
    dom = max(rows, key=lambda r: r["ms"])
    if args.layers:
        for r in rows:
            print(f"{r['layer']:>10s} {r['op']:>9s} {r['ms']*1e3:9.1f} us  {r['bound']:>4s}  {100*r['frac']:6.2f}% of peak",
                  file=sys.stderr)
        print(f"sum of kernels {total_ms:.3f} ms; graph step {ms_per_step:.3f} ms", file=sys.stderr)
    if dom["bound"] == "mfma":
        roof = {"bound": "mfma", "achieved": dom["work"] / (dom["ms"] * 1e-3) / 1e12, "peak": INT8_MFMA_PEAK_OPS / 1e12,
                "unit": "TOP/s"}
    else:
        roof = {"bound": "hbm", "achieved": dom["work"] / (dom["ms"] * 1e-3) / 1e9, "peak": HBM_PEAK_BYTES / 1e9,
                "unit": "GB/s"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    roof["traffic"] = None
    roof["kernel"] = f"{dom['layer']} ({dom['op']}), {dom['ms']*1e3:.1f} us of {total_ms*1e3:.1f} us"

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
        "config": {"workload": f"{net.name} int8 (QAsymm activations, per-channel QSymmS8 weights), batch {batch}, "
                               f"random-init, whole forward pass incl. avgpool/FC/softmax, input resident in HBM",
                   "batch": batch, "graph_replay": not args.no_graph, "fused_depthwise_pointwise": args.fuse,
                   "total_TOPS": 2.0 * net.macs_per_image() * batch / (ms_per_step * 1e-3) / 1e12},
        "roofline": roof, "groups": groups,
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(net)
    dn.close()
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
