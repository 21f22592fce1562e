"""Layer chains (one persistent launch for a run of layers) against layer-by-layer launches (needs an MI355X)."""
import numpy as np
import pytest

from armnn_amd import nets, shim
from armnn_amd.executor import DeviceNetwork

pytestmark = pytest.mark.gpu


def _chain_equals_layers(net, batch, lanes=1, replays=3, **kw):
    """Every tensor a chain writes, on every replay (fresh input each time), equals what separate launches write."""
    plain = DeviceNetwork(net, batch, use_graph=False, lanes=1)
    chained = DeviceNetwork(net, batch, use_graph=True, lanes=lanes, chain=True, **kw)
    runs = [l for l, _ in chained.steps if getattr(l, "op", "") == "chain"]
    assert runs, "no chain was formed"
    print(f"{net.name} b{batch}: chains", [(r.name, len(r.parts)) + c.info() for r, c in zip(runs, chained.chains)], flush=True)
    for r in range(replays):
        x = nets.synthetic_input(net, batch, seed=100 + r)
        want = plain.run(x)
        got = chained.run(x)
        assert sum(c.gave_up() for c in chained.chains) == 0
        for run in runs:
            for l in run.parts:
                a = plain.download(l.output).data
                b = chained.download(l.output).data
                bad = int((a != b).sum())
                assert bad == 0, f"replay {r}: {l.name}: {bad} of {a.size} bytes differ"
        np.testing.assert_array_equal(got.data, want.data)
    plain.close()
    chained.close()


def test_mobilenet_chain_batch2():
    _chain_equals_layers(nets.mobilenet_v1(), 2)


def test_mobilenet_chain_batch8_two_lanes():
    _chain_equals_layers(nets.mobilenet_v1(), 8, lanes=2)


def test_mobilenet_chain_batch64():
    _chain_equals_layers(nets.mobilenet_v1(), 64, lanes=2, replays=4)


def test_mobilenet_chain_batch64_lanes_after_chain():
    _chain_equals_layers(nets.mobilenet_v1(), 64, lanes=2, replays=2, lanes_after_chain=True)


def test_mobilenet_chain_odd_resolution_batch3():
    # ragged tiles: 160 x 160 input gives 10 x 10 and 5 x 5 maps
    _chain_equals_layers(nets.mobilenet_v1(resolution=160), 3)


@pytest.mark.parametrize("option, value, default, batch", [
    (b"chain_stages", 3, 2, 4), (b"chain_stages", 4, 2, 4),
    (b"chain_blocks_per_cu", 1, 0, 4),
    (b"chain_defer_signal", 1, 0, 8),      # tiles counted as finished behind the next tile's loads
    (b"chain_panel", 1, 0, 40),            # batch 40: enough row blocks for the resident-panel work items (28 x 28 and 14 x 14 layers)
])
def test_mobilenet_chain_variants(option, value, default, batch):
    lib = shim.load_library()
    shim._chk(lib.mi355x_set_option(option, value))
    try:
        _chain_equals_layers(nets.mobilenet_v1(), batch, replays=2)
    finally:
        shim._chk(lib.mi355x_set_option(option, default))


def test_chain_refuses_what_it_cannot_run():
    """Layers outside the chain's envelope and tensors that overlap are answered with an error, not run."""
    net = nets.mobilenet_v1()
    dn = DeviceNetwork(net, 2, use_graph=False)
    plans = {l.name: p for (l, _), p in zip(dn.steps, dn._step_plans)}
    assert not shim.LayerChain.accepts(plans["stem"], 2)          # 3 input channels
    assert not shim.LayerChain.accepts(plans["pw1"], 2)           # 32 input channels: the weight-stationary kernel's layout
    assert shim.LayerChain.accepts(plans["dw7"], 2) and shim.LayerChain.accepts(plans["pw7"], 2)
    x, mid, out = (dn.buffers[n].ptr for n in (dn.net.layers[13].inputs[0], dn.net.layers[13].output, dn.net.layers[14].output))
    l13, l14 = dn.net.layers[13], dn.net.layers[14]
    assert (l13.name, l14.name) == ("dw7", "pw7")
    with pytest.raises(shim.ShimError, match="overlap"):
        shim.LayerChain([plans["dw7"], plans["pw7"]], 2, x, [mid, x])          # the run's output over its input
    with pytest.raises(shim.ShimError, match="does not consume"):
        shim.LayerChain([plans["pw7"], plans["dw5"]], 2, x, [mid, out])
    dn.close()
