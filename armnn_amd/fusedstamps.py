"""Phase timings of the fused depthwise + pointwise kernel (measurement support).

    make -C armnn_amd/csrc stamps
    python -m armnn_amd.fusedstamps [--batch 64] [--pair dw7+pw7]

Loads the measurement build of the device library, whose DwPwPanelKernel records wave 0's shader-clock stamps per block;
its 40th launch prints to stderr the average cycles between consecutive stamps over all blocks: prologue, then per
128-channel block the depthwise phase, the wait for the weights plus the block barrier, and the GEMM phase, then the
requantization of the output tile and its stores."""
from __future__ import annotations

import argparse
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--pair", default="dw7+pw7")
    args = ap.parse_args()
    from armnn_amd import shim
    lib = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libarmnn_mi355x_stamps.so")
    if not os.path.exists(lib):
        raise SystemExit(f"{lib} not found: build it with `make -C armnn_amd/csrc stamps`")
    shim.load_library(lib)
    from armnn_amd import nets
    from armnn_amd.executor import DeviceNetwork
    net = nets.mobilenet_v1()
    dn = DeviceNetwork(net, args.batch, use_graph=False, lanes=1, fuse="dwpw")
    dn.run(nets.synthetic_input(net, args.batch))
    for l, fn in dn.steps:
        if l.name == args.pair:
            for _ in range(45):
                fn(dn.stream)
            dn.synchronize()
            break
    else:
        raise SystemExit(f"no fused step named {args.pair}: " + ", ".join(l.name for l, _ in dn.steps if getattr(l, "op", "") == "dwpw"))
    dn.close()


if __name__ == "__main__":
    main()
