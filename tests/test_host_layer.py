"""Runs the C++ test driver of the host layer (tests/host/test_main.cc): the reference-style
build -> lower -> routine tests of the plugin surface (collectors, kernels, Device, MemPool,
Resources).  The `cpu` part needs no GPU; the `gpu` part runs every routine on the AMD device and
checks it against the CPU oracle."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
EXE = os.path.join(HERE, "host", "_build", "rg_host_tests")


def _run(mode):
    if not os.path.exists(EXE):
        pytest.fail(f"{EXE} not built: run `make -C tests/host` (or __graft_entry__.build())")
    proc = subprocess.run([EXE, mode], capture_output=True, text=True, timeout=300)
    print(proc.stdout[-4000:], proc.stderr[-2000:])
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
    assert " 0 failed" in proc.stdout


def test_host_layer_logic_cpu():
    _run("cpu")


@pytest.mark.gpu
def test_host_layer_routines_on_gpu():
    _run("gpu")
