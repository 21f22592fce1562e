"""Runs a nets.Network layer by layer on the CPU checker -- TEST INFRASTRUCTURE ONLY.

Fused activations are applied the way CpuRef sees them: as a separate Activation layer after the producing
layer, with the same quantization in and out."""
from __future__ import annotations

from typing import Dict, Optional

from armnn_amd.nets import Network
from armnn_amd.tensor import QTensor

from .cpuref import Oracle


def run_network(orc: Oracle, net: Network, x: QTensor, keep: bool = False, fast: bool = True,
                overrides: Optional[Dict[str, QTensor]] = None):
    """Returns the output tensor, or every tensor by name when keep=True.  `overrides` replaces the input of a
    layer by a given tensor (used to judge each layer on identical inputs)."""
    batch = x.info.shape[0]
    vals: Dict[str, QTensor] = {net.input: x}
    for l in net.layers:
        ins = [vals[i] for i in l.inputs]
        out_info = net.info(l.output, batch)
        if l.op in ("conv", "depthwise"):
            p = {k: v for k, v in l.params.items() if not k.startswith("_")}
            y = orc.conv2d(ins[0], l.weights, l.bias, out_info, fast=fast, **p)
        elif l.op == "fc":
            y = orc.fully_connected(ins[0], l.weights, l.bias, out_info, transpose_weights=l.params["transpose_weights"], fast=fast)
        elif l.op == "pool":
            y = orc.pooling2d(ins[0], out_info, **l.params)
        elif l.op == "add":
            y = orc.add(ins[0], ins[1], out_info)
        elif l.op == "activation":
            y = orc.activation(ins[0], out_info, l.act[0], l.act[1], l.act[2])
        elif l.op == "pad":
            y = orc.pad(ins[0], out_info, [b for b, _ in l.params["pad_list"]], l.params["pad_value"])
        elif l.op == "softmax":
            y = orc.softmax(ins[0], out_info, l.params["beta"], -1)
        elif l.op == "reshape":
            y = QTensor(out_info, ins[0].data.reshape(out_info.shape))
        else:
            raise ValueError(l.op)
        if l.act[0] and l.op != "activation":
            y = orc.activation(y, out_info, l.act[0], l.act[1], l.act[2])
        vals[l.output] = y
    return vals if keep else vals[net.output]
