#!/usr/bin/env python3
"""Benchmark: int8 images/sec of the MobileNetV1-1.0-224-style network at batch 64 on one MI355X.

A step is one forward pass of the whole network over one batch that is already resident in HBM (every layer
runs on the device through the C ABI; the pass reaches the device as one replay of a captured HIP graph or kernel by
kernel on the stream, whichever a trial before the warm-up steps finds faster: --submission, config.submission_trial).
Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 64] [--net mobilenet_v1|resnet50]
                  [--weights per_channel_s8|per_tensor_u8] [--no-cpu-baseline] [--no-backend] [--layers] [--chain]
                  [--submission auto|graph|eager]

The headline workload is the default: per-channel QSymmS8 weights.  --weights per_tensor_u8 runs the same network with
QAsymmU8 weights that have one scale and a zero point per layer, and says so in config.workload.

Extra objects in the line:
  roofline      the kernel SYMBOL with the largest summed time over one step: algorithmic work of all its launches over
                their summed time (each launch HIP-event timed alone on the launch stream), `traffic` = the summed counter
                bytes of those launches from the committed rocprofv3 summary (null when the profile was taken with other
                kernels than run now); roofline_next holds the next two symbols
  config.backend_path   the same network through IRuntime::EnqueueWorkload on the C++ backend (child process, wall clock,
                host buffers in and out: pageable, and pinned buffers adopted with ImportInputs / ImportOutputs); its output
                bytes are compared with the executor's
  groups        conv/FC ops vs the int8 MFMA peak and depthwise bytes vs the HBM peak over the whole net
  cpu_baseline  the reference's CpuRef backend behind its own runtime where that build is there, else the reference's own
                CpuRef functions (oracle/_ref) -- both kind "reference" -- or the C restatement (kind "port"); one thread, on a
                bounded sample of the same workload
  parity        the timed device network run once more, outside the timed region, on the images the cpu_baseline leg
                computed: max |difference| in codes and exact-match fraction against the CPU checker, end to end, for the
                network's output and for the logits in front of the softmax
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

TRAFFIC_PROFILES = {
    # (network name, images per launch) -> rocprofv3 counter summary written by `python -m armnn_amd.profile_summary traffic`
    ("mobilenet_v1_1.0_224", 64): os.path.join(ROOT, "profiles", "mobilenet_v1_b64_hbm_traffic.md"),
    ("resnet50_224", 16): os.path.join(ROOT, "profiles", "resnet50_b32_hbm_traffic.md"),
}


def measured_traffic(net_name, launch_batch):
    """{layer: (kernel name, HBM bytes read + written per launch)} from the committed counter summary of this workload
    (FETCH_SIZE and WRITE_SIZE passes, each scaled by a calibration copy; the file says how it was made), or {}."""
    path = TRAFFIC_PROFILES.get((net_name, launch_batch))
    table = {}
    if not path or not os.path.exists(path):
        return table
    with open(path) as f:
        for line in f:
            cells = [c.strip() for c in line.strip().strip("|").split("|")]
            if len(cells) >= 5 and cells[1].startswith("`"):
                try:
                    table[cells[0]] = (cells[1].strip("`"), float(cells[4]) * 1e6)
                except ValueError:
                    pass
    return table


def layer_work(net, l, batch):
    """(kind, algorithmic work per launch): conv/fc -> ops = 2*MACs; others -> bytes, each tensor once."""
    if l.op in ("conv", "fc"):
        return "mfma", 2.0 * l.macs_per_image * batch
    if l.op in ("convadd", "convpool"):        # a convolution with the Addition / the global pooling behind it in its write-out
        return "mfma", 2.0 * l.parts[0].macs_per_image * batch
    if l.op in ("chain", "tail"):
        # a run of layers in one persistent launch: every layer's tensors are still written and read, so the launch's
        # algorithmic bytes are the sum of its layers'; priced against HBM like the depthwise layers in it
        return "hbm", float(sum(algorithmic_bytes(net, part, batch) for part in l.parts))
    if l.op == "dwpw":
        # two layers fused (depthwise + pointwise, in either order): the tensor between them never exists, so the unit's
        # algorithmic bytes are its input, its output and both layers' constants; priced against HBM like the depthwise
        # layer it absorbs
        first, second = l.parts
        nbytes = (net.tensors[first.inputs[0]].num_elements + net.tensors[second.output].num_elements) * batch
        for part in (first, second):
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


def cpu_baseline_reference_runtime(net, seconds_budget=25.0):
    """The same network at batch 1 through IRuntime::EnqueueWorkload on the reference's own CpuRef backend: backend_bench
    built against the reference's source tree and the libarmnn.so made from it (armnn_amd/backend/test/bin/real/).  None
    when that build is not there."""
    import subprocess
    import tempfile
    import numpy as np
    from armnn_amd import netfile, nets
    exe = os.path.join(ROOT, "armnn_amd", "backend", "test", "bin", "real", "backend_bench")
    if not os.path.exists(exe):
        return None
    with tempfile.TemporaryDirectory(prefix="mi355x_cpuref_") as tmp:
        nf, fin, fout = (os.path.join(tmp, n) for n in ("net.bin", "input.bin", "output.bin"))
        netfile.write_net(net, 1, nf)
        np.ascontiguousarray(nets.synthetic_input(net, 1, seed=100).data).tofile(fin)
        images, elapsed = 0, 0.0
        steps = 1
        while True:
            try:
                r = subprocess.run([exe, nf, fin, fout, str(steps), "0", "CpuRef"], capture_output=True, text=True, timeout=600)
            except subprocess.TimeoutExpired:
                return None
            if r.returncode != 0:
                return None
            ms = json.loads(r.stdout.strip().splitlines()[-1])["ms_pageable"]
            images += steps
            elapsed += steps * ms * 1e-3
            if elapsed * (images + steps) / images > seconds_budget or images >= 8:
                break
        info = net.info(net.output, 1)
        from armnn_amd.tensor import numpy_dtype
        outputs = [(100, {net.output: np.fromfile(fout, dtype=numpy_dtype(info.dtype)).reshape(info.shape)})]
    return {"_outputs": outputs, "value": images / elapsed, "unit": "images/sec", "cores": 1, "kind": "reference",
            "sample": f"{images} image(s) of the same network at batch 1 through IRuntime::EnqueueWorkload on the reference's CpuRef backend "
                      f"(libarmnn.so built from the reference), {elapsed:.1f} s, single-threaded backend on one of {os.cpu_count()} cores"}


def cpu_baseline(net, seconds_budget=25.0):
    real = cpu_baseline_reference_runtime(net, seconds_budget)
    if real is not None:
        return real
    from oracle import cpuref, netref
    from armnn_amd import nets
    kind = "reference" if cpuref.have("reference") else "port"
    if kind == "port" and not cpuref.have("port"):
        cpuref.build(reference=False)
    orc = cpuref.Oracle(kind)
    os.environ["OMP_NUM_THREADS"] = "1"
    images, elapsed = 0, 0.0
    outputs = []
    keep = {net.output, net.layers[-1].inputs[0]}       # the network's output and what the last layer reads (the logits)
    while True:
        x = nets.synthetic_input(net, 1, seed=100 + images)
        t0 = time.perf_counter()
        vals = netref.run_network(orc, net, x, fast=False, keep=True)      # literal single-thread loop nest, as CpuRef runs it
        elapsed += time.perf_counter() - t0
        outputs.append((100 + images, {k: vals[k].data for k in keep}))
        images += 1
        if elapsed * (images + 1) / images > seconds_budget or images >= 8:
            break
    return {"_outputs": outputs, "value": images / elapsed, "unit": "images/sec", "cores": 1, "kind": kind,
            "sample": f"{images} image(s) of the same network at batch 1, {elapsed:.1f} s, 1 thread of {os.cpu_count()}"}


def parity_against_checker(net, dn, batch, checked):
    """The timed device network (same plans, same graph) run once more on a batch whose first images are the ones the CPU
    baseline computed, outside the timed region; the CPU side is the checker only.  End to end: differences of the layers
    add up along the network, so max_abs_lsb here is not the per-layer bound the tests assert (<= 1 per layer on
    identical inputs, armnnTestUtils/TensorHelpers.hpp:24-31 is the reference's own tolerance rule)."""
    import numpy as np
    from armnn_amd import nets
    x = nets.synthetic_input(net, batch)
    for k, (seed, _) in enumerate(checked[:batch]):
        x.data[k] = nets.synthetic_input(net, 1, seed=seed).data[0]
    dn.upload_input(x)
    dn.enqueue()
    out = {"images": min(len(checked), batch), "against": "CPU checker outputs of the cpu_baseline leg, end to end"}
    for name in checked[0][1]:
        got = dn.download(name).data
        d = np.concatenate([np.abs(got[k].astype(np.int32) - ref[name][0].astype(np.int32)).ravel() for k, (_, ref) in enumerate(checked[:batch])])
        key = "output" if name == net.output else "logits"
        out[key] = {"tensor": name, "max_abs_lsb": int(d.max()), "exact_fraction": float((d == 0).mean()), "within_1_lsb_fraction": float((d <= 1).mean())}
    if "output" in out:
        out["max_abs_lsb"], out["exact_fraction"] = out["output"]["max_abs_lsb"], out["output"]["exact_fraction"]
    return out


def run_backend_child(net, batch, steps, warmup, real=False, lanes=0):
    """The same network through the C++ backend (INetwork -> Optimize -> LoadNetwork -> IRuntime::EnqueueWorkload) in a
    child process, started before this process has touched the GPU.  Returns (figures, output bytes) or (error, None).
    real=True runs the build of the same program against an Arm NN source tree and its own libarmnn.so
    (armnn_amd/backend/test/bin/real/, made by `make -C armnn_amd/backend real-runtime`), if it is there.
    lanes > 0 sets the backend's lane count for the child (environment variable MI355X_LANES, which the backend reads once)."""
    import subprocess
    import tempfile
    import numpy as np
    from armnn_amd import netfile, nets
    exe = os.path.join(ROOT, "armnn_amd", "backend", "test", "bin", *(["real"] if real else []), "backend_bench")
    if not os.path.exists(exe):
        return {"error": os.path.relpath(exe, ROOT) + " is not built"}, None
    with tempfile.TemporaryDirectory(prefix="mi355x_bench_") as tmp:
        nf, fin, fout = (os.path.join(tmp, n) for n in ("net.bin", "input.bin", "output.bin"))
        netfile.write_net(net, batch, nf)
        np.ascontiguousarray(nets.synthetic_input(net, batch).data).tofile(fin)
        try:
            env = dict(os.environ)
            if lanes > 0:
                env["MI355X_LANES"] = str(lanes)
            r = subprocess.run([exe, nf, fin, fout, str(steps), str(warmup)], capture_output=True, text=True, timeout=300, env=env)
        except subprocess.TimeoutExpired:
            return {"error": "backend_bench timed out"}, None
        if r.returncode != 0:
            return {"error": f"backend_bench exit {r.returncode}: {r.stderr.strip()[-300:]}"}, None
        fig = json.loads(r.stdout.strip().splitlines()[-1])
        if lanes > 0:
            fig["lanes"] = lanes
        with open(fout, "rb") as f:
            return fig, f.read()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3000, help="timed forward passes (the default keeps the timed region above a second)")
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--net", default="mobilenet_v1", choices=["mobilenet_v1", "resnet50"])
    ap.add_argument("--weights", default="per_channel_s8", choices=["per_channel_s8", "per_tensor_u8"],
                    help="mobilenet_v1 only: per_tensor_u8 gives every layer QAsymmU8 weights with one scale and a zero point "
                         "(the quantization of older uint8 models) instead of the headline workload's per-channel QSymmS8")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-backend", action="store_true", help="skip the run through the C++ backend (config.backend_path)")
    ap.add_argument("--no-graph", action="store_true", help="launch every pass kernel by kernel (same as --submission eager)")
    ap.add_argument("--submission", default="auto", choices=("auto", "graph", "eager"),
                    help="how a forward pass reaches the device: one replay of the captured HIP graph, kernel by kernel on the stream, or "
                         "(auto) whichever of the two is faster in a trial of 2 x 40 passes each before the warm-up steps")
    ap.add_argument("--fuse", default="auto", choices=("auto", "none", "dwpw", "pwdw"),
                    help="pairs of layers as one kernel (same bytes): 'auto' the depthwise + pointwise pairs the library recommends at "
                         "the batch a launch sees (mi355x_conv2d_fusion_pays), 'none' every layer a launch of its own, 'dwpw' every "
                         "depthwise + pointwise pair the fused kernels accept, 'pwdw' pointwise + the depthwise after it where whole images fit a block")
    ap.add_argument("--fuse-tail", action="store_true", help="pooling, FullyConnected and Softmax at the end of the network as one launch instead of three (same bytes, measured slower)")
    ap.add_argument("--no-fuse-add", action="store_true",
                    help="launch a residual Addition on its own instead of inside the convolution that feeds it")
    ap.add_argument("--lanes", type=int, default=0,
                    help="split the batch into this many slices, each running the network on a stream of its own "
                         "(default: 2 for batches of at least 16 images that halve, else 1)")
    ap.add_argument("--chain", action="store_true",
                    help="runs of consecutive layers the library accepts (3x3 depthwise over multiples of 128 channels, 1x1 convolutions "
                         "over more than 128 input channels) as one persistent launch over the whole batch (same bytes)")
    ap.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                    help="mi355x_set_option before any plan is created (tests and tuning), e.g. igemm_xcd_cols=1")
    ap.add_argument("--layers", action="store_true", help="print the per-layer table to stderr")
    ap.add_argument("--profile-pass", action="store_true",
                    help="for rocprofv3 --pmc: one 64 MiB calibration copy (1 B read + 1 B written per element), then ONE "
                         "eager forward pass, one kernel per layer in network order; prints the dispatch order as JSON")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus N with N > 1 is not supported "
              "(the path shards by batch with no exchange step: one process per GPU would run the same plans on its slice).", file=sys.stderr)
        return 2

    from armnn_amd import nets
    net = nets.mobilenet_v1(weights=args.weights) if args.net == "mobilenet_v1" else nets.resnet50()
    batch = args.batch

    # ---- the product path north_star names: the backend behind IRuntime::EnqueueWorkload, in a child process that is
    # started (and has ended) before anything here touches the GPU
    if args.lanes == 0:
        # Two lanes overlap the tails of one lane's launches with the other's; the 3x3 depthwise kernel sizes its grid to
        # the whole device and walks its items itself, and two of those side by side get in each other's way
        # (MobileNetV1, 64 images: 0.330 ms in one lane, 0.336 in two; ResNet-50, 32 images: 0.864 and 0.725).
        depthwise = any(l.op == "depthwise" for l in net.layers)
        args.lanes = 2 if batch >= 16 and batch % 2 == 0 and not depthwise else 1
    backend, backend_out = (None, None)
    real, real_out = (None, None)
    if not args.no_backend and not args.profile_pass:
        # (the backend with the executor's lane count: through EnqueueWorkload MobileNetV1 b64 takes 0.306 ms in one lane
        # against 0.327 in two with input and output resident)
        backend, backend_out = run_backend_child(net, batch, max(50, args.steps // 4), 20, lanes=args.lanes)
        real, real_out = run_backend_child(net, batch, max(50, args.steps // 4), 20, real=True, lanes=args.lanes)

    from armnn_amd import shim
    from armnn_amd.executor import DeviceNetwork

    for opt in args.option:
        name, _, value = opt.partition("=")
        shim.set_option(name, int(value))
    if args.no_graph:
        args.submission = "eager"
    dn = DeviceNetwork(net, batch, use_graph=args.submission != "eager", fuse="" if args.fuse == "none" else args.fuse, lanes=args.lanes, fuse_add=not args.no_fuse_add, chain=args.chain, fuse_tail=args.fuse_tail)
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
        kernels = []
        for _, fn in dn.steps:
            fn(dn.stream, 0, args.lanes)                 # lane 0's launch of every layer, as the timed region launches it
            kernels.append(dn.lib.mi355x_last_kernel().decode(errors="replace"))
        dev.stream_sync(dn.stream)
        print(json.dumps({"dispatch_order": ["fill (setup)", f"calibration copy {n} B in + {n} B out"] + [l.name for l, _ in dn.steps],
                          "kernels": ["FillU8Kernel", "ActivationKernel"] + kernels,
                          "algorithmic_bytes": [n, 2 * n] + [algorithmic_bytes(net, l, batch // args.lanes) for l, _ in dn.steps],
                          "batch": batch, "launch_batch": batch // args.lanes, "net": net.name}))
        dn.close()
        return 0

    # ---- set-up: which way of submitting a pass is faster here (like a plan's choice of kernel, made once, before the warm-up)
    submission = dn.choose_submission() if args.submission == "auto" else None

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
    executor_out = dn.download().data.tobytes()

    # ---- per-kernel timing on the launch stream, for the roofline object ------------------------------------
    # (one launch = one layer over one lane's slice of the batch; in the timed region `lanes` such launches of a layer
    # run side by side on their own streams)
    launch_batch = batch // args.lanes
    per_layer = dn.time_layers(iters=50, warmup=10)
    traffic = measured_traffic(net.name, launch_batch)
    rows = []
    for l, ms, kernel in per_layer:
        images = batch if l.op == "chain" else launch_batch        # a layer chain runs the whole batch in one launch
        kind, work = layer_work(net, l, images)
        peak = INT8_MFMA_PEAK_OPS if kind == "mfma" else HBM_PEAK_BYTES
        row = {"layer": l.name, "op": l.op, "ms": ms, "bound": kind, "work": work, "frac": work / (ms * 1e-3) / peak, "kernel": kernel}
        if kind == "mfma":
            # the roof that binds a conv / FC layer depends on its arithmetic intensity: below the ridge
            # (peak ops / peak bytes = 625 ops/B) the HBM roof is the lower one
            nbytes = float(algorithmic_bytes(net, l, images))
            row["bytes"] = nbytes
            row["ops"] = work
            row["binding"] = "mfma" if work / nbytes >= RIDGE_OPS_PER_BYTE else "hbm"
        else:
            row["bytes"] = work
            row["ops"] = 0.0
            row["binding"] = "hbm"
        # counter bytes of this layer's launch, only while the profile was taken with the kernel that runs now
        t = traffic.get(l.name)
        row["traffic"] = t[1] if t and t[0] == kernel else None
        rows.append(row)
    total_ms = sum(r["ms"] for r in rows)
    if args.layers:
        for r in rows:
            hbm = r["bytes"] / (r["ms"] * 1e-3) / HBM_PEAK_BYTES
            print(f"{r['layer']:>10s} {r['op']:>9s} {r['ms']*1e3:9.1f} us  {r['bound']:>4s} {100*r['frac']:6.2f}% of peak"
                  f"   binding roof {r['binding']:>4s}, {100*hbm:5.1f}% of HBM peak on algorithmic bytes   {r['kernel']}", file=sys.stderr)
        print(f"launches of {launch_batch} images; sum of one lane's launches {total_ms:.3f} ms; step of {args.lanes} lane(s) "
              f"{ms_per_step:.3f} ms", file=sys.stderr)

    # ---- the dominant kernel: the symbol with the largest summed time over one step
    by_kernel = {}
    for r in rows:
        by_kernel.setdefault(r["kernel"], []).append(r)

    def kernel_roof(name):
        sel = by_kernel[name]
        t = sum(r["ms"] for r in sel) * 1e-3
        ops, nbytes = sum(r["ops"] for r in sel), sum(r["bytes"] for r in sel)
        mfma_bound = ops > 0 and ops / nbytes >= RIDGE_OPS_PER_BYTE
        if mfma_bound:
            roof = {"bound": "mfma", "achieved": ops / t / 1e12, "peak": INT8_MFMA_PEAK_OPS / 1e12, "unit": "TOP/s"}
        else:
            roof = {"bound": "hbm", "achieved": nbytes / t / 1e9, "peak": HBM_PEAK_BYTES / 1e9, "unit": "GB/s"}
        roof["frac"] = roof["achieved"] / roof["peak"]
        roof["traffic"] = sum(r["traffic"] for r in sel) if all(r["traffic"] is not None for r in sel) else None
        roof["kernel"] = name
        roof["launches_per_lane_pass"] = len(sel)
        roof["layers"] = [r["layer"] for r in sel]
        roof["avg_launch_us"] = t * 1e6 / len(sel)
        roof["share_of_lane_pass"] = t * 1e3 / total_ms
        roof["algorithmic_bytes"] = nbytes
        roof["timing"] = ("HIP events around repeated launches of each layer alone on the stream, same buffers every time: every tensor of a "
                          "launch fits the 256 MB last-level cache, so fractions of the HBM roof are upper bounds on what HBM itself sees")
        if ops > 0:
            roof["TOPS"] = ops / t / 1e12
            roof["frac_of_int8_mfma_peak"] = ops / t / INT8_MFMA_PEAK_OPS
        return roof

    ranked = sorted(by_kernel, key=lambda k: -sum(r["ms"] for r in by_kernel[k]))
    roof = kernel_roof(ranked[0])
    runners_up = [kernel_roof(k) for k in ranked[1:3]]

    def group(ops, peak):
        sel = [r for r in rows if r["op"] in ops]
        t = sum(r["ms"] for r in sel) * 1e-3
        w = sum(r["work"] for r in sel)
        return {"ms": t * 1e3, "achieved": w / t, "frac": w / t / peak} if t > 0 else None

    g_conv = group(("conv", "fc", "convadd", "convpool"), INT8_MFMA_PEAK_OPS)
    g_dw = group(("depthwise",), HBM_PEAK_BYTES)
    groups = {
        "conv_fc": {"ms": g_conv["ms"], "TOPS": g_conv["achieved"] / 1e12, "frac_of_int8_mfma_peak": g_conv["frac"]},
    }
    if g_dw:
        groups["depthwise"] = {"ms": g_dw["ms"], "GBps": g_dw["achieved"] / 1e9, "frac_of_hbm_peak": g_dw["frac"]}
    fused_rows = [r for r in rows if r["op"] == "dwpw"]
    if fused_rows:
        # depthwise + pointwise pairs that ran as one launch belong to neither group above: their time buys both the pointwise
        # layer's ops and the pair's bytes (input, output, constants; the tensor between the layers never exists)
        t = sum(r["ms"] for r in fused_rows) * 1e-3
        by_name = {l.name: l for l, _, _ in per_layer}
        ops = sum(2.0 * next(part for part in by_name[r["layer"]].parts if part.op == "conv").macs_per_image * launch_batch for r in fused_rows)
        nbytes = sum(r["work"] for r in fused_rows)
        groups["fused_depthwise_pointwise"] = {"ms": t * 1e3, "launches": len(fused_rows), "TOPS": ops / t / 1e12, "frac_of_int8_mfma_peak": ops / t / INT8_MFMA_PEAK_OPS,
                                               "GBps": nbytes / t / 1e9, "frac_of_hbm_peak": nbytes / t / HBM_PEAK_BYTES}

    config = {"workload": f"{net.name} int8 (QAsymm activations, {'per-channel QSymmS8' if args.weights == 'per_channel_s8' or args.net != 'mobilenet_v1' else 'per-tensor QAsymmU8'} weights), batch {batch}, "
                          f"random-init, whole forward pass incl. avgpool/FC/softmax, input resident in HBM, every layer through the C ABI, "
                          + ("one HIP graph replay per step" if dn.use_graph else "the kernels of a step launched one by one on the stream"),
              "batch": batch, "graph_replay": bool(dn.use_graph), "submission_trial": submission, "fused_pairs": [l.name for l, _ in dn.steps if l.op == "dwpw"] or None, "additions_inside_convolutions": not args.no_fuse_add, "lanes": args.lanes,
              "layer_chains": [l.name for l, _ in dn.steps if l.op == "chain"] or None,
              "tail_in_one_launch": any(l.op == "tail" for l, _ in dn.steps),
              "convolution_and_global_pooling_in_one_launch": [l.name for l, _ in dn.steps if l.op == "convpool"] or None,
              "total_TOPS": 2.0 * net.macs_per_image() * batch / (ms_per_step * 1e-3) / 1e12}
    if backend is not None:
        # the same network and input through the C++ backend: wall clock per IRuntime::EnqueueWorkload call, host buffers in
        # and out (PCIe inclusive; never `value`)
        bp = dict(backend)
        if backend_out is not None:
            bp["output_equals_executor"] = backend_out == executor_out
            bp["images_per_sec_pageable_io"] = batch / (backend["ms_pageable"] * 1e-3)
            bp["images_per_sec_adopted_pinned_io"] = batch / (backend["ms_pinned"] * 1e-3)
            if backend.get("ms_device_resident"):
                bp["images_per_sec_device_resident_io"] = batch / (backend["ms_device_resident"] * 1e-3)
            bp["path"] = "INetwork -> Optimize({Mi355x}) -> IRuntime::LoadNetwork -> IRuntime::EnqueueWorkload (armnn_amd/backend/test/BackendBench.cpp)"
        if real is not None and real_out is not None:
            # the same program built against the reference's source tree: the reference's own optimizer, loaded network and
            # runtime drive the backend
            bp["reference_runtime"] = {"ms_pageable": real["ms_pageable"], "ms_pinned": real["ms_pinned"],
                                       "ms_device_resident": real.get("ms_device_resident"),
                                       "output_equals_executor": real_out == executor_out,
                                       "images_per_sec_pageable_io": batch / (real["ms_pageable"] * 1e-3),
                                       "images_per_sec_adopted_pinned_io": batch / (real["ms_pinned"] * 1e-3),
                                       "optimized_layers": real["optimized_layers"], "activation_layers_left": real["activation_layers_left"],
                                       "memcopy_layers": real["memcopy_layers"],
                                       "path": "the same calls on libarmnn.so built from the reference's sources (armnn_amd/backend/test/bin/real/backend_bench)"}
        elif real is not None:
            bp["reference_runtime"] = real
        config["backend_path"] = bp

    line = {
        "metric": f"int8 images/sec MobileNetV1 b{batch} @1 GPU" if args.net == "mobilenet_v1" else f"int8 images/sec {args.net} b{batch} @1 GPU",
        "value": images_per_s, "unit": "images/sec", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": config,
        "roofline": roof, "roofline_next": runners_up, "groups": groups,
    }
    # what the device itself delivers on register-only MFMA chains and on a plain copy, next to the published peaks
    from armnn_amd import peaks
    line["measured_peaks"] = peaks.measure()
    if not args.no_cpu_baseline:
        base = cpu_baseline(net)
        checked = base.pop("_outputs", [])
        line["cpu_baseline"] = base
        if checked:
            line["parity"] = parity_against_checker(net, dn, batch, checked)
    dn.close()
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
