"""Runs a nets.Network on the device through the C ABI: one plan per layer, all activations resident in HBM,
the whole forward pass launched kernel by kernel or captured into a HIP graph and replayed with one launch
(DeviceNetwork.choose_submission measures which is faster for the network and batch at hand)."""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import numpy as np

from . import shim
from .nets import Network
from .tensor import QTensor, numpy_dtype


@dataclass
class FusedPair:
    """Two neighbouring layers -- depthwise + the pointwise convolution consuming it, pointwise + the depthwise consuming
    it, a convolution + the Addition consuming it (op "convadd"), or a 1x1 convolution + the pooling over its whole output
    image (op "convpool") -- launched as one kernel."""
    name: str
    parts: Tuple                       # (first Layer, second Layer)
    op: str = "dwpw"

    @property
    def inputs(self):
        return tuple(self.parts[0].inputs) + tuple(i for i in self.parts[1].inputs if i != self.parts[0].output)

    @property
    def output(self):
        return self.parts[1].output

    @property
    def macs_per_image(self):
        return self.parts[0].macs_per_image + self.parts[1].macs_per_image


@dataclass
class ChainedRun:
    """Consecutive convolution layers executed by one persistent launch (shim.LayerChain) over the whole batch."""
    name: str
    parts: Tuple                       # the Layers, in order
    op: str = "chain"

    @property
    def inputs(self):
        return tuple(self.parts[0].inputs)

    @property
    def output(self):
        return self.parts[-1].output

    @property
    def macs_per_image(self):
        return sum(p.macs_per_image for p in self.parts)


@dataclass
class FusedTail:
    """Global pooling, the FullyConnected layer behind it and the Softmax behind that, executed by one launch
    (shim.ClassifierTail); all three tensors are still written."""
    name: str
    parts: Tuple                       # (pooling Layer, FullyConnected Layer, Softmax Layer)
    op: str = "tail"

    @property
    def inputs(self):
        return tuple(self.parts[0].inputs)

    @property
    def output(self):
        return self.parts[-1].output

    @property
    def macs_per_image(self):
        return self.parts[1].macs_per_image


class DeviceNetwork:
    def __init__(self, net: Network, batch: int, algo_overrides: Optional[Dict[str, int]] = None, use_graph: bool = True,
                 fuse: bool = False, lanes: int = 1, fuse_add: bool = True, chain: bool = False, lanes_after_chain: bool = False,
                 join_for_fused: bool = False, fuse_tail: bool = False, fuse_pool: Optional[bool] = None):
        """fuse_pool: a 1x1 convolution and the pooling over its whole output image as one launch (Conv2dPlan.run_pooled; same
        bytes, the convolution's output tensor is not written): True wherever the library takes the pair, None (default) where
        it also recommends it and fuse == "auto", False never.
        fuse_tail: global pooling -> FullyConnected -> Softmax at the end of the network as one launch (same bytes; measured
        slower than the three launches on MI355X, so off by default).
        chain: runs of consecutive layers the library accepts (mi355x_chain_accepts) become one persistent launch over
        the whole batch; with lanes > 1 the lanes join in front of such a run and, if lanes_after_chain, fork again behind it
        (else the rest of the network runs on one stream).
        lanes > 1 splits the batch into that many contiguous slices; each slice runs the whole network on a stream of
        its own (the same plans, pointers offset to the slice), so one slice's kernels fill the ramp-up, tail and
        launch gaps of the others. Results do not depend on the split: every image is computed independently."""
        if lanes < 1 or batch % lanes != 0:
            raise ValueError("lanes must divide the batch")
        self.net, self.batch = net, batch
        self.lanes = lanes
        self.dev = shim.Device()
        self.lib = shim.load_library()
        self.stream = self.dev.stream()
        self.side_streams = [self.dev.stream() for _ in range(lanes - 1)]
        self.buffers: Dict[str, shim.DeviceBuffer] = {}
        self.steps: List = []          # (layer, callable(stream))
        self._step_plans: List = []    # plan of each step (None for plan-less layers), parallel to self.steps
        self.plans = []
        self.chains: List = []
        self.tails: List = []
        self._pool_descs = {}
        self.lanes_after_chain = lanes_after_chain
        self.join_for_fused = join_for_fused      # fused pairs run on the whole batch: the lanes join in front of the first one
        self.graph = None
        self.use_graph = use_graph
        algo_overrides = algo_overrides or {}

        def buf(name):
            if name not in self.buffers:
                self.buffers[name] = shim.DeviceBuffer(net.info(name, batch).num_elements)
            return self.buffers[name]

        buf(net.input)
        for l in net.layers:
            xin = [net.info(i, batch) for i in l.inputs]
            yout = net.info(l.output, batch)
            if l.op == "reshape":
                self.buffers[l.output] = self.buffers[l.inputs[0]]      # same bytes, new shape
                continue
            xb = [buf(i) for i in l.inputs]
            yb = buf(l.output)
            if l.op in ("conv", "depthwise"):
                p = {k: v for k, v in l.params.items() if not k.startswith("_")}
                plan = shim.Conv2dPlan(xin[0], l.weights, l.bias, yout, activation=l.act[0], act_a=l.act[1],
                                       act_b=l.act[2], algo=algo_overrides.get(l.name, shim.ALGO_AUTO), **p)
                plan.set_concurrency(lanes)
                self.plans.append(plan)
                self.steps.append((l, self._conv_step(plan, xb[0].ptr, yb.ptr, xin[0].num_elements, yout.num_elements)))
                self._step_plans.append(plan)
            elif l.op == "fc":
                plan = shim.FullyConnectedPlan(xin[0], l.weights, l.bias, yout, transpose_weights=l.params["transpose_weights"],
                                               activation=l.act[0], act_a=l.act[1], act_b=l.act[2],
                                               algo=algo_overrides.get(l.name, shim.ALGO_AUTO))
                self.plans.append(plan)
                self.steps.append((l, self._conv_step(plan, xb[0].ptr, yb.ptr, xin[0].num_elements, yout.num_elements)))
                self._step_plans.append(plan)
            elif l.op == "pool":
                _, h, w, c = xin[0].shape
                _, ho, wo, _ = yout.shape
                p = l.params
                d = shim.Pool2dDesc(h, w, c, ho, wo, p["pool_w"], p["pool_h"], p["stride_x"], p["stride_y"], p["pad_left"],
                                    p["pad_right"], p["pad_top"], p["pad_bottom"], p["pool_type"], p["padding_method"],
                                    shim._quant(xin[0]), shim._quant(yout))
                self._pool_descs[id(l)] = d
                self.steps.append((l, self._pool_step(d, xb[0].ptr, yb.ptr, xin[0].num_elements, yout.num_elements, l.act,
                                                      shim._quant(yout))))
                self._step_plans.append(None)
            elif l.op == "add":
                q0, q1, qo = shim._quant(xin[0]), shim._quant(xin[1]), shim._quant(yout)
                self.steps.append((l, self._add_step(yout.num_elements, q0, q1, qo, l.act, xb[0].ptr, xb[1].ptr, yb.ptr)))
                self._step_plans.append(None)
            elif l.op == "activation":
                qi, qo = shim._quant(xin[0]), shim._quant(yout)
                self.steps.append((l, self._activation_step(yout.num_elements, qi, qo, l.act, xb[0].ptr, yb.ptr)))
                self._step_plans.append(None)
            elif l.op == "pad":
                self.steps.append((l, self._pad_step(xin[0], yout, l.params["pad_list"], l.params["pad_value"], xb[0].ptr, yb.ptr)))
                self._step_plans.append(None)
            elif l.op == "softmax":
                rows, cols = yout.shape
                qi, qo = shim._quant(xin[0]), shim._quant(yout)
                self.steps.append((l, self._softmax_step(rows, cols, l.params["beta"], qi, qo, xb[0].ptr, yb.ptr)))
                self._step_plans.append(None)
            else:
                raise ValueError(l.op)
        self._plan_of = {id(l): pl for (l, _), pl in zip(self.steps, self._step_plans)}
        if fuse in ("dwpw", "pwdw", True):
            self._fuse_pairs(("conv", "depthwise") if fuse == "pwdw" else ("depthwise", "conv"))
        elif fuse == "auto":
            # only the pairs the library recommends as one launch at the batch a launch sees
            self._fuse_pairs(("depthwise", "conv"), only_where_it_pays=True)
            # ... and, among the layers still on their own, 1x1 convolution + the depthwise layer behind it where recommended
            self._fuse_pairs(("conv", "depthwise"), only_where_it_pays=True)
        if fuse_add:
            self._fuse_additions()
        if chain:
            self._build_chains()
        if fuse_tail:
            self._fuse_tail()
        if fuse_pool or (fuse_pool is None and fuse == "auto"):
            self._fuse_conv_pool(only_where_it_pays=not fuse_pool)

    def _fuse_conv_pool(self, only_where_it_pays):
        """A 1x1 convolution whose output only feeds the pooling launched right behind it, where the library runs the two
        as one kernel (mi355x_conv2d_pool_fusable): the step writes the pooled tensor only."""
        net = self.net
        consumers: Dict[str, int] = {}
        for l in net.layers:
            for i in l.inputs:
                consumers[i] = consumers.get(i, 0) + 1
        fused, k = [], 0
        while k < len(self.steps):
            l, fn = self.steps[k]
            nxt = self.steps[k + 1][0] if k + 1 < len(self.steps) else None
            plan = self._plan_of.get(id(l)) if getattr(l, "op", None) == "conv" else None
            d = self._pool_descs.get(id(nxt)) if getattr(nxt, "op", None) == "pool" else None
            rows = self.batch // self.lanes
            if (isinstance(plan, shim.Conv2dPlan) and d is not None and nxt.inputs[0] == l.output and nxt.act[0] == 0 and
                    consumers.get(l.output, 0) == 1 and l.output != net.output and plan.pool_fusable(d) and
                    (not only_where_it_pays or plan.pool_fusion_pays(d, rows))):
                x, y = self.buffers[l.inputs[0]].ptr, self.buffers[nxt.output].ptr
                nx, ny = net.info(l.inputs[0], self.batch).num_elements, net.info(nxt.output, self.batch).num_elements
                batch = self.batch
                fused.append((FusedPair(f"{l.name}+{nxt.name}", (l, nxt), op="convpool"),
                              (lambda plan, d, x, y, nx, ny: lambda s, lane=0, lanes=1: plan.run_pooled(
                                  d, batch // lanes, x + lane * (nx // lanes), y + lane * (ny // lanes), s))(plan, d, x, y, nx, ny)))
                k += 2
            else:
                fused.append((l, fn))
                k += 1
        self.steps = fused

    def _fuse_tail(self):
        """Pooling over the whole image -> FullyConnected -> Softmax, launched one behind the other, become one launch where
        the library takes the three (mi355x_tail_create); each lane gets an object of its own, because launches of one
        object must not overlap."""
        net, batch, lanes = self.net, self.batch, self.lanes
        rows = batch // lanes
        k = 0
        while k + 2 < len(self.steps):
            (lp, _), (lf, _), (ls, _) = self.steps[k:k + 3]
            if not (getattr(lp, "op", None) == "pool" and getattr(lf, "op", None) == "fc" and getattr(ls, "op", None) == "softmax" and
                    lp.act[0] == 0 and self.buffers[lf.inputs[0]] is self.buffers[lp.output] and ls.inputs[0] == lf.output):
                k += 1
                continue
            fc_plan = self._plan_of[id(lf)]
            cols = net.info(lf.output, batch).shape[-1]
            chans = net.info(lp.output, batch).shape[-1]
            if (rows * cols) % 4 != 0:
                k += 1
                continue
            try:
                tails = [shim.ClassifierTail(self._pool_descs[id(lp)], fc_plan, ls.params["beta"], net.info(ls.output, batch))
                         for _ in range(lanes)]
            except shim.ShimError:
                k += 1
                continue
            self.tails.extend(tails)
            x, pooled = self.buffers[lp.inputs[0]].ptr, self.buffers[lp.output].ptr
            logits, y = self.buffers[lf.output].ptr, self.buffers[ls.output].ptr
            nx = net.info(lp.inputs[0], batch).num_elements

            def fn(s, lane=0, lanes=1, tails=tails, x=x, pooled=pooled, logits=logits, y=y, nx=nx, chans=chans, cols=cols):
                r = batch // lanes
                tails[lane].run(r, x + lane * (nx // lanes), pooled + lane * r * chans, logits + lane * r * cols, y + lane * r * cols, s)
            self.steps[k:k + 3] = [(FusedTail(f"{lp.name}+{lf.name}+{ls.name}", (lp, lf, ls)), fn)]
            k += 1

    def _build_chains(self, min_layers: int = 2):
        """Replace every maximal run of consecutive steps that are plain convolution / depthwise layers accepted by the
        library, each reading the output of the one before, by one chain step."""
        plan_of = self._plan_of
        batch = self.batch

        def eligible(step):
            l = step[0]
            return (getattr(l, "op", None) in ("conv", "depthwise") and isinstance(plan_of.get(id(l)), shim.Conv2dPlan) and
                    shim.LayerChain.accepts(plan_of[id(l)], batch))

        out, k = [], 0
        while k < len(self.steps):
            if not eligible(self.steps[k]):
                out.append(self.steps[k])
                k += 1
                continue
            run = [self.steps[k]]
            while (k + len(run) < len(self.steps) and eligible(self.steps[k + len(run)]) and
                   self.steps[k + len(run)][0].inputs[0] == run[-1][0].output):
                run.append(self.steps[k + len(run)])
            if len(run) < min_layers:
                out.append(self.steps[k])
                k += 1
                continue
            layers = [st[0] for st in run]
            ch = shim.LayerChain([plan_of[id(l)] for l in layers], batch, self.buffers[layers[0].inputs[0]].ptr,
                                 [self.buffers[l.output].ptr for l in layers])
            self.chains.append(ch)

            def fn(s, lane=0, lanes=1, ch=ch):
                ch.run(s)
            fn.whole_batch = True
            out.append((ChainedRun("chain(" + layers[0].name + ".." + layers[-1].name + ")", tuple(layers)), fn))
            k += len(run)
        self.steps = out

    def _fuse_pairs(self, ops, only_where_it_pays=False):
        """Replace neighbours (depthwise 3x3, 1x1 convolution) -- or, with ops = ("conv", "depthwise"), (1x1 convolution,
        depthwise 3x3) -- by one fused launch where the library accepts the pair and nothing else reads the tensor
        between them."""
        net = self.net
        consumers: Dict[str, int] = {}
        for l in net.layers:
            for i in l.inputs:
                consumers[i] = consumers.get(i, 0) + 1
        plan_of = self._plan_of
        fused, k = [], 0
        while k < len(self.steps):
            l, fn = self.steps[k]
            nxt = self.steps[k + 1][0] if k + 1 < len(self.steps) else None
            if (l.op == ops[0] and nxt is not None and nxt.op == ops[1] and nxt.inputs[0] == l.output and
                    consumers.get(l.output, 0) == 1 and l.output != net.output and
                    plan_of[id(l)].fusable_with(plan_of[id(nxt)]) and
                    (not only_where_it_pays or plan_of[id(l)].fusion_pays(plan_of[id(nxt)], self.batch if self.join_for_fused else self.batch // self.lanes))):
                pdw, ppw = plan_of[id(l)], plan_of[id(nxt)]
                x, y = self.buffers[l.inputs[0]].ptr, self.buffers[nxt.output].ptr
                nx, ny = net.info(l.inputs[0], self.batch).num_elements, net.info(nxt.output, self.batch).num_elements
                batch = self.batch
                if self.join_for_fused and self.lanes > 1:
                    fn2 = (lambda pdw, ppw, x, y: lambda s, lane=0, lanes=1: pdw.run_fused(ppw, batch, x, y, s))(pdw, ppw, x, y)
                    fn2.whole_batch = True
                else:
                    fn2 = (lambda pdw, ppw, x, y, nx, ny: lambda s, lane=0, lanes=1: pdw.run_fused(
                        ppw, batch // lanes, x + lane * (nx // lanes), y + lane * (ny // lanes), s))(pdw, ppw, x, y, nx, ny)
                fused.append((FusedPair(f"{l.name}+{nxt.name}", (l, nxt)), fn2))
                k += 2
            else:
                fused.append((l, fn))
                k += 1
        self.steps = fused

    def _fuse_additions(self):
        """A convolution whose output only feeds the Addition launched right behind it (the last convolution of a residual
        block) runs that Addition inside its own write-out (Conv2dPlan.run_add): same bytes, one launch and one round trip
        of the tensor less.  The Addition's other input was produced earlier, so launch order is unchanged."""
        net = self.net
        consumers: Dict[str, int] = {}
        for l in net.layers:
            for i in l.inputs:
                consumers[i] = consumers.get(i, 0) + 1
        plan_of = self._plan_of
        fused, k = [], 0
        while k < len(self.steps):
            l, fn = self.steps[k]
            nxt = self.steps[k + 1][0] if k + 1 < len(self.steps) else None
            if (l.op == "conv" and nxt is not None and nxt.op == "add" and l.output in nxt.inputs and nxt.inputs[0] != nxt.inputs[1] and
                    consumers.get(l.output, 0) == 1 and l.output != net.output and isinstance(plan_of.get(id(l)), shim.Conv2dPlan)):
                plan = plan_of[id(l)]
                other = nxt.inputs[1] if nxt.inputs[0] == l.output else nxt.inputs[0]
                x, o, y = self.buffers[l.inputs[0]].ptr, self.buffers[other].ptr, self.buffers[nxt.output].ptr
                nx, ny = net.info(l.inputs[0], self.batch).num_elements, net.info(nxt.output, self.batch).num_elements
                oi, si = net.info(other, self.batch), net.info(nxt.output, self.batch)
                batch, act = self.batch, nxt.act
                fused.append((FusedPair(f"{l.name}+{nxt.name}", (l, nxt), op="convadd"),
                              (lambda plan, x, o, y, nx, ny, oi, si, act: lambda s, lane=0, lanes=1: plan.run_add(
                                  batch // lanes, x + lane * (nx // lanes), o + lane * (ny // lanes), oi, si, y + lane * (ny // lanes),
                                  activation=act[0], act_a=act[1], act_b=act[2], stream=s))(plan, x, o, y, nx, ny, oi, si, act)))
                k += 2
            else:
                fused.append((l, fn))
                k += 1
        self.steps = fused

    # each step keeps its ctypes structs alive through the closure
    # A step is callable(stream, lane=0, lanes=1): lane k of n works on images [k*batch/n, (k+1)*batch/n) of every buffer.
    def _conv_step(self, plan, x, y, nx, ny):
        batch = self.batch
        return lambda s, lane=0, lanes=1: plan.run(batch // lanes, x + lane * (nx // lanes), y + lane * (ny // lanes), s)

    def _pool_step(self, d, x, y, nx, ny, act=(0, 0.0, 0.0), qo=None):
        """Pooling, then -- when the layer carries a fused activation, as a parsed AVERAGE_POOL_2D / MAX_POOL_2D may
        (src/armnnTfLiteParser/TfLiteParser.cpp ParsePool -> AddFusedActivationLayer) -- the activation in place on the
        pooled tensor, in the output's own quantization."""
        batch, lib = self.batch, self.lib

        def run(s, lane=0, lanes=1):
            out = y + lane * (ny // lanes)
            shim._chk(lib.mi355x_pool2d_run(C.byref(d), batch // lanes, x + lane * (nx // lanes), out, s))
            if act[0] != 0:
                shim._chk(lib.mi355x_activation_run(ny // lanes, C.byref(qo), C.byref(qo), act[0], act[1], act[2], out, out, s))
        return run

    def _add_step(self, n, q0, q1, qo, act, x0, x1, y):
        lib = self.lib
        return lambda s, lane=0, lanes=1: shim._chk(lib.mi355x_add_run(
            n // lanes, C.byref(q0), C.byref(q1), C.byref(qo), act[0], act[1], act[2], x0 + lane * (n // lanes),
            x1 + lane * (n // lanes), y + lane * (n // lanes), s))

    def _activation_step(self, n, qi, qo, act, x, y):
        lib = self.lib
        return lambda s, lane=0, lanes=1: shim._chk(lib.mi355x_activation_run(
            n // lanes, C.byref(qi), C.byref(qo), act[0], act[1], act[2], x + lane * (n // lanes), y + lane * (n // lanes), s))

    def _pad_step(self, xin, yout, pad_list, pad_value, x, y):
        lib = self.lib
        nx, ny = xin.num_elements, yout.num_elements
        batch_padded = tuple(pad_list[0]) != (0, 0)
        descs = {}

        def run(s, lane=0, lanes=1):
            if batch_padded and lanes > 1:
                raise ValueError("a Pad layer that pads the batch cannot run in lanes")
            if lanes not in descs:
                shape = (xin.shape[0] // lanes,) + tuple(xin.shape[1:])
                descs[lanes] = shim.pad_desc(shape, pad_list, pad_value, xin, yout)
            shim._chk(lib.mi355x_pad_run(C.byref(descs[lanes]), x + lane * (nx // lanes), y + lane * (ny // lanes), s))
        return run

    def _softmax_step(self, rows, cols, beta, qi, qo, x, y):
        lib = self.lib
        return lambda s, lane=0, lanes=1: shim._chk(lib.mi355x_softmax_run(
            rows // lanes, cols, beta, C.byref(qi), C.byref(qo), x + lane * (rows // lanes) * cols,
            y + lane * (rows // lanes) * cols, s))

    # ---------------------------------------------------------------------------------------------------------
    def upload_input(self, x: QTensor):
        assert x.info.shape == self.net.info(self.net.input, self.batch).shape
        self.buffers[self.net.input].upload(x.data, self.stream)

    def _enqueue_lanes(self):
        """Every lane's chain of launches: lane 0 on self.stream, the others on streams forked from it and joined back.
        A step that works on the whole batch (a layer chain) runs on self.stream with the lanes joined in front of it."""
        if self.lanes == 1:
            for _, fn in self.steps:
                fn(self.stream)
            return
        forked = False
        single_from_here = False

        def fork():
            ev = self._sync_event()
            self.dev.event_record(ev, self.stream)
            for side in self.side_streams:
                self.dev.stream_wait_event(side, ev)

        def join():
            for side in self.side_streams:
                ev = self._sync_event()
                self.dev.event_record(ev, side)
                self.dev.stream_wait_event(self.stream, ev)

        self._sync_next = 0
        # lanes interleaved layer by layer, so launches next to each other in submission order can overlap
        for _, fn in self.steps:
            if getattr(fn, "whole_batch", False) or single_from_here:
                if forked:
                    join()
                    forked = False
                fn(self.stream, 0, 1)
                if getattr(fn, "whole_batch", False) and not self.lanes_after_chain:
                    single_from_here = True
                continue
            if not forked:
                fork()
                forked = True
            fn(self.stream, 0, self.lanes)
            for k, side in enumerate(self.side_streams, start=1):
                fn(side, k, self.lanes)
        if forked:
            join()

    def _sync_event(self):
        """Events for forks and joins, one per use within a forward pass (a captured graph keeps them)."""
        if not hasattr(self, "_sync_events"):
            self._sync_events, self._sync_next = [], 0
        if self._sync_next == len(self._sync_events):
            self._sync_events.append(self.dev.event())
        ev = self._sync_events[self._sync_next]
        self._sync_next += 1
        return ev

    def enqueue(self):
        """One forward pass on self.stream (asynchronous)."""
        if self.use_graph:
            if self.graph is None:
                self.dev.graph_begin(self.stream)
                self._enqueue_lanes()
                self.graph = self.dev.graph_end(self.stream)
            self.dev.graph_launch(self.graph, self.stream)
        else:
            self._enqueue_lanes()

    def choose_submission(self, passes: int = 40, rounds: int = 2):
        """Times `passes` forward passes launched kernel by kernel and the same number of replays of the captured graph,
        alternated `rounds` times, and keeps the faster way for enqueue() (self.use_graph).  A replay costs the host one call,
        so it wins where the host cannot launch as fast as the device computes (a few images per pass); at tens of images
        per pass the device is the limit, and there kernels launched one by one on the stream finish a few percent sooner
        than the same kernels as nodes of a graph.  Returns {"eager_ms", "graph_ms"}: the best pass time of either way."""
        import time
        best = {False: float("inf"), True: float("inf")}
        for _ in range(rounds):
            for mode in (False, True):
                self.use_graph = mode
                self.enqueue()                         # first use captures the graph
                self.synchronize()
                t0 = time.perf_counter()
                for _ in range(passes):
                    self.enqueue()
                self.synchronize()
                best[mode] = min(best[mode], (time.perf_counter() - t0) * 1e3 / passes)
        self.use_graph = best[True] < best[False]
        self.submission = {"eager_ms": best[False], "graph_ms": best[True]}
        return self.submission

    def synchronize(self):
        self.dev.stream_sync(self.stream)

    def download(self, name: Optional[str] = None) -> QTensor:
        name = name or self.net.output
        info = self.net.info(name, self.batch)
        self.synchronize()
        return QTensor(info, self.buffers[name].download(info.shape, numpy_dtype(info.dtype), self.stream))

    def run(self, x: QTensor) -> QTensor:
        self.upload_input(x)
        self.enqueue()
        return self.download()

    def time_layers(self, iters: int = 20, warmup: int = 3):
        """(layer, device time in ms of one launch, kernel name) of every step, as launched by enqueue() (lane 0's slice
        of the batch when the network runs in lanes), alone on the launch stream, timed with HIP events on that stream.
        The kernel name is what the library reports for the step's last launch (mi355x_last_kernel)."""
        e0, e1 = self.dev.event(), self.dev.event()
        out = []
        for l, fn in self.steps:
            for _ in range(warmup):
                fn(self.stream, 0, self.lanes)
            self.dev.event_record(e0, self.stream)
            for _ in range(iters):
                fn(self.stream, 0, self.lanes)
            self.dev.event_record(e1, self.stream)
            self.dev.event_sync(e1)
            kernel = self.lib.mi355x_last_kernel().decode(errors="replace")
            out.append((l, self.dev.elapsed_ms(e0, e1) / iters, kernel))
        return out

    def close(self):
        if self.graph is not None:
            self.dev.graph_destroy(self.graph)
            self.graph = None
        for ch in self.chains:
            ch.destroy()
        self.chains = []
        for t in self.tails:
            t.destroy()
        self.tails = []
        for p in self.plans:
            p.destroy()
        for b in set(self.buffers.values()):
            b.free()
        for side in self.side_streams:
            self.dev.stream_destroy(side)
        self.dev.stream_destroy(self.stream)
