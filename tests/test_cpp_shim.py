"""Runs the C++ test program of the host-side operator shim
(include/cut_hip_ops.hpp, mirror of DequantOpNode / MatMulOpNode of the
reference).  The binary is built by `make -C tests/cpp` (part of build())."""
import os
import subprocess

import pytest

BIN = os.path.join(os.path.dirname(__file__), "cpp", "host_shim_test")


def _run(mode):
    if not os.path.exists(BIN):
        pytest.fail(f"{BIN} is not built: run `make -C tests/cpp` (or __graft_entry__.build())")
    r = subprocess.run([BIN, mode], capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stdout + r.stderr


def test_shim_tables_and_validation_cpu():
    _run("--cpu")


@pytest.mark.gpu
def test_shim_nodes_against_oracle_gpu():
    _run("--gpu")
