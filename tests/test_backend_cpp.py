"""The C++ side of the boundary: the Mi355x backend behind the Arm NN backend interfaces.

The cases themselves are C++ (armnn_amd/backend/test/*.cpp) because the interfaces are C++; this module runs the two
test executables and fails on any failed case.  "cpu" cases exercise host logic only (registry, layer support,
descriptor validation, fusion, arena planning, no-device behaviour, dynamic loading); "gpu" cases run networks through
INetwork -> Optimize -> LoadNetwork -> EnqueueWorkload on the device and compare with the CPU oracle.
"""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BACKEND = os.path.join(ROOT, "armnn_amd", "backend")
BIN = os.path.join(BACKEND, "test", "bin")


def _ensure_built():
    need = [os.path.join(BIN, "backend_tests"), os.path.join(BIN, "dynamic_tests"), os.path.join(BIN, "backend_bench"),
            os.path.join(ROOT, "armnn_amd", "lib", "Amd_Mi355x_backend.so")]
    if all(os.path.exists(p) for p in need):
        return
    import __graft_entry__
    __graft_entry__.build()


def _run(exe, tag, timeout):
    _ensure_built()
    proc = subprocess.run([os.path.join(BIN, exe), "--tag", tag], capture_output=True, text=True, timeout=timeout)
    print(proc.stdout)
    print(proc.stderr)
    assert proc.returncode == 0, f"{exe} --tag {tag} failed:\n{proc.stdout[-4000:]}\n{proc.stderr[-2000:]}"
    assert " 0 failed" in proc.stdout
    ran = int(proc.stdout.strip().splitlines()[-1].split()[0])
    assert ran > 0, "no case ran"
    return proc.stdout


def test_backend_host_logic():
    out = _run("backend_tests", "cpu", 300)
    assert "registry: Mi355x is registered" in out


def test_backend_dynamic_loading_host():
    _run("dynamic_tests", "cpu", 300)


@pytest.mark.gpu
def test_backend_networks_on_device():
    out = _run("backend_tests", "gpu", 600)
    assert "max |diff|" in out


@pytest.mark.gpu
def test_backend_dynamic_on_device():
    _run("dynamic_tests", "gpu", 300)


@pytest.mark.gpu
@pytest.mark.parametrize("runtime", ["host_core", "reference_runtime"])
@pytest.mark.parametrize("name,batch", [("resnet50", 32), ("mobilenet_v1", 64)])
def test_benchmark_network_through_the_backend_equals_the_executor(tmp_path, name, batch, runtime):
    """ResNet-50 at batch 32 (7x7 stem, max pooling, 16 residual adds with their ReLU folded in, 53 convolutions) and
    MobileNetV1 at batch 64, from one network file: INetwork -> Optimize({Mi355x}) -> LoadNetwork -> EnqueueWorkload in
    backend_bench gives the bytes the C-ABI executor gives (which the network tests tie to the CPU checker), with pageable
    and with adopted pinned host buffers; no Activation layer survives optimization and no copy layer is inserted.
    "reference_runtime" is the same program built against an Arm NN source tree and run on the libarmnn.so made from it:
    the reference's optimizer, LoadedNetwork and Runtime around this backend."""
    import json

    import numpy as np

    from armnn_amd import netfile, nets
    from armnn_amd.executor import DeviceNetwork

    _ensure_built()
    exe = os.path.join(BIN, "backend_bench") if runtime == "host_core" else os.path.join(BIN, "real", "backend_bench")
    if runtime == "reference_runtime" and not os.path.exists(exe):
        pytest.skip("the backend has not been built against an Arm NN source tree (make -C armnn_amd/backend real-armnn real-runtime)")
    assert os.path.exists(exe), "backend_bench is not built"
    net = nets.resnet50() if name == "resnet50" else nets.mobilenet_v1()
    x = nets.synthetic_input(net, batch, seed=11)
    nf, fin, fout = (str(tmp_path / n) for n in ("net.bin", "input.bin", "output.bin"))
    netfile.write_net(net, batch, nf)
    np.ascontiguousarray(x.data).tofile(fin)
    proc = subprocess.run([exe, nf, fin, fout, "20", "3"], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
    fig = json.loads(proc.stdout.strip().splitlines()[-1])
    print(f"{name} b{batch} through EnqueueWorkload ({runtime}): {fig['ms_pageable']:.3f} ms pageable I/O = {batch / fig['ms_pageable'] * 1e3:.0f} images/s, "
          f"{fig['ms_pinned']:.3f} ms adopted pinned I/O = {batch / fig['ms_pinned'] * 1e3:.0f} images/s; {fig}", flush=True)
    assert fig["pinned_equals_pageable"] and fig["activation_layers_left"] == 0 and fig["memcopy_layers"] == 0
    assert fig["add_layers"] == (16 if name == "resnet50" else 0)
    # every residual Addition of ResNet-50 runs the convolution in front of it inside its own launch
    assert fig["additions_running_a_convolution"] == fig["add_layers"]
    dn = DeviceNetwork(net, batch, use_graph=False)
    want = dn.run(x).data.tobytes()
    dn.close()
    with open(fout, "rb") as f:
        got = f.read()
    assert got == want, "the backend's output differs from the executor's"


@pytest.mark.skipif(not os.path.isdir("/root/reference/include/armnn"), reason="needs an Arm NN source tree")
def test_backend_sources_compile_against_real_armnn_headers():
    """-fsyntax-only against the reference's own headers: the backend uses no name the real API lacks."""
    proc = subprocess.run(["make", "-C", BACKEND, "conformance"], capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stdout[-3000:] + proc.stderr[-3000:]


REAL = os.path.join(BIN, "real")


def _real_runtime():
    """Runs test/bin/real/real_runtime_tests: libarmnn.so built from an Arm NN source tree loads the backend, compiled
    against that tree's headers, from a dynamic backend directory."""
    exe = os.path.join(REAL, "real_runtime_tests")
    if not os.path.exists(exe):
        pytest.skip("the backend has not been built against an Arm NN source tree (make -C armnn_amd/backend real-armnn real-runtime)")
    proc = subprocess.run([exe, os.path.join(REAL, "backends")], capture_output=True, text=True, timeout=300)
    out = proc.stdout
    print("\n".join(l for l in out.splitlines() if not l.startswith("optimizer:")))
    print(proc.stderr[-2000:])
    assert proc.returncode == 0, out[-4000:]
    assert " 0 failed" in out and "registered backends: CpuRef, Mi355x" in out
    return out


def test_backend_in_the_real_runtime_host():
    """The reference's own runtime finds Amd_Mi355x_backend.so by name, accepts its API version and registers Mi355x; the
    backend's id, capabilities and layer support answer through the public handles; on a machine without the device
    the backend context is unavailable, every layer is refused with the reason, Optimize({Mi355x, CpuRef}) places the
    network on CpuRef and the runtime computes it; the runtime's destructor deregisters the backend."""
    import shutil
    if os.path.isdir("/root/reference/include/armnn") and os.path.exists(os.environ.get("ARMNN_BUILD", "/tmp/mi355x_armnn_build") + "/libarmnn.so") \
            and shutil.which("make"):
        proc = subprocess.run(["make", "-C", BACKEND, "real-runtime"], capture_output=True, text=True, timeout=900)
        assert proc.returncode == 0, proc.stdout[-3000:] + proc.stderr[-3000:]
    out = _real_runtime()
    from armnn_amd import shim
    if shim.Device.count() == 0:
        assert "backend context unavailable" in out and "random convolution on CpuRef" in out
        assert "IsConvolution2dSupported(QAsymmS8 NHWC 3x3): no" in out


@pytest.mark.gpu
def test_backend_in_the_real_runtime_on_device():
    """The same executable where there is a device: the reference's runtime creates the backend context, the optimizer
    places every layer on Mi355x, and the outputs are within one code of what the reference's CpuRef backend computes in
    the same process (convolution, strided depthwise, pointwise, pooling, reshape, fully connected, folded activations)."""
    out = _real_runtime()
    assert "backend context created" in out
    assert "random convolution on Mi355x against CpuRef" in out
    assert "fully connected on Mi355x against CpuRef" in out
