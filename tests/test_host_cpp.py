"""The C++ host layer (ROCm memory manager, device context, bundle helpers)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SELFTEST = os.path.join(ROOT, "execution-ucx_amd", "lib", "host_selftest")
REFERENCE = "/root/reference"


def test_host_layer_without_device(pkg):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    assert os.path.exists(SELFTEST), "build the host self-test with `make -C execution-ucx_amd host`"
    out = subprocess.run([SELFTEST, "--no-device"], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "host_selftest ok" in out.stdout


def test_host_layer_compiles_against_the_reference_headers():
    """Only where the execution-ucx tree is mounted (never on the GPU box)."""
    if not os.path.exists(os.path.join(REFERENCE, "ucx_context", "ucx_context_data.hpp")):
        pytest.skip("reference tree not present")
    cmd = ["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-DAXON_ROCM_IN_REFERENCE_TREE",
           "-I", REFERENCE, "-I", os.path.join(ROOT, "include"),
           "-I", os.path.join(ROOT, "execution-ucx_amd", "host"),
           os.path.join(ROOT, "tests", "cpp", "in_tree_compile_check.cpp")]
    out = subprocess.run(cmd, capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr


@pytest.mark.gpu
def test_host_layer_on_device(gpu):
    out = subprocess.run([SELFTEST], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "host_selftest ok" in out.stdout
