"""The chain entry point that allocates nothing against the chain object's launch (needs an MI355X).
Collected last on purpose: every call on a GPU shares one device array."""
import numpy as np
import pytest

from armnn_amd import nets, shim
from armnn_amd.executor import DeviceNetwork

pytestmark = pytest.mark.gpu


def _back_half(dn):
    """(plans, input pointer, output pointers, layers) of the network's longest run of chain members."""
    plans, layers = [], []
    best = ([], [])
    for (l, _), p in zip(dn.steps, dn._step_plans):
        ok = isinstance(p, shim.Conv2dPlan) and shim.LayerChain.accepts(p, dn.batch) and (not layers or l.inputs[0] == layers[-1].output)
        if ok:
            plans.append(p); layers.append(l)
        else:
            if len(layers) > len(best[1]):
                best = (plans, layers)
            plans, layers = ([p], [l]) if isinstance(p, shim.Conv2dPlan) and shim.LayerChain.accepts(p, dn.batch) else ([], [])
    if len(layers) > len(best[1]):
        best = (plans, layers)
    plans, layers = best
    return plans, dn.buffers[layers[0].inputs[0]].ptr, [dn.buffers[l.output].ptr for l in layers], layers


def test_chain_without_allocation_equals_the_chain_object_twice_in_a_row():
    net = nets.mobilenet_v1()
    for batch, seed in ((16, 41), (6, 42)):               # the second call is the smaller one: the array keeps the first one's contents
        dn = DeviceNetwork(net, batch, use_graph=False, lanes=1)
        x = nets.synthetic_input(net, batch, seed=seed)
        dn.run(x)                                          # every layer by its own launch: fills the run's input tensor
        plans, x_dev, outs, layers = _back_half(dn)
        assert len(layers) >= 10
        chain = shim.LayerChain(plans, batch, x_dev, outs)
        chain.run(dn.stream)
        dn.synchronize()
        assert chain.gave_up() == 0
        want = [dn.download(l.output).data.copy() for l in layers]
        for l in layers:                                   # wipe, so that stale bytes cannot pass
            shim._chk(dn.lib.mi355x_fill_u8(dn.buffers[l.output].ptr, 0x5a, dn.net.info(l.output, batch).num_elements, dn.stream))
        shim.LayerChain.run_noalloc(plans, batch, x_dev, outs, dn.stream)
        dn.synchronize()
        for l, w in zip(layers, want):
            got = dn.download(l.output).data
            assert np.array_equal(got, w), f"batch {batch}: {l.name} differs"
        chain.destroy()
        dn.close()


def test_chain_without_allocation_rejects_what_exceeds_its_array():
    net = nets.mobilenet_v1()
    dn = DeviceNetwork(net, 2, use_graph=False)
    plans, x_dev, outs, layers = _back_half(dn)
    with pytest.raises(shim.ShimError, match="at most 32 layers and 64 images"):
        shim.LayerChain.run_noalloc(plans, 65, x_dev, outs, dn.stream)
    with pytest.raises(shim.ShimError, match="at most 32 layers and 64 images"):
        shim.LayerChain.run_noalloc(plans * 3, 2, x_dev, outs * 3, dn.stream)
    dn.close()
