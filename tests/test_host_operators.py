"""The host-side mirror of the reference's operator interface (parameter-server_amd/host/): a C++
driver replays the reference's test_sparse flow through wire-format requests. Needs an MI355X."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(HERE, "cpp", "test_hbm_operators")


@pytest.mark.gpu
def test_operator_mirror_replays_test_sparse(tmp_path):
    assert os.path.exists(BINARY), "build it with __graft_entry__.build() (make -C tests/cpp)"
    r = subprocess.run([BINARY, str(tmp_path)], capture_output=True, text=True, timeout=100)
    print(r.stdout[-2000:], r.stderr[-2000:])
    assert r.returncode == 0 and "PASS test_hbm_operators" in r.stdout


def test_operator_mirror_compiles_without_prpc():
    """hbm_ops.h needs nothing but the C ABI header and the stand-in types (no GPU needed)."""
    src = os.path.join(HERE, "cpp", "test_hbm_operators.cpp")
    r = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-Wextra", src],
                       capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stderr[-2000:]
