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
    need = [os.path.join(BIN, "backend_tests"), os.path.join(BIN, "dynamic_tests"),
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


@pytest.mark.skipif(not os.path.isdir("/root/reference/include/armnn"), reason="needs an Arm NN source tree")
def test_backend_sources_compile_against_real_armnn_headers():
    """-fsyntax-only against the reference's own headers: the backend uses no name the real API lacks."""
    proc = subprocess.run(["make", "-C", BACKEND, "conformance"], capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stdout[-3000:] + proc.stderr[-3000:]
