"""The C ABI called from plain C++ (tests/cabi/layer_cli.cpp: HIP-runtime allocations, no Python,
no torch): a fused and a per-operator encoder layer against the CPU oracle."""
import json
import os
import subprocess

import pytest

from gpu_util import announce

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "cabi", "layer_cli.bin")


def test_cli_is_built_and_links_the_library():
    assert os.path.exists(BIN), "build it with __graft_entry__.build() or make -C tests/cabi"
    out = subprocess.run(["ldd", BIN], capture_output=True, text=True).stdout
    assert "libsouffle_hip.so" in out and "not found" not in out, out


@pytest.mark.gpu
def test_plain_cpp_caller_matches_oracle():
    announce("C ABI from plain C++")
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stdout + r.stderr
    res = json.loads(r.stdout.strip().splitlines()[-1])
    assert res["ok"] and res["max_abs"] <= 2e-2 and res["mean_abs"] <= 2e-3
