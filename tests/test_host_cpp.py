"""The C++17 host mirror (motifcl_amd/host: Tensor / Backend / nn::CounterStateLinear over the
C ABI) and its test executables, which restate MotifCL's own counter tests
(tests/test_vulkan_counter_fused.cpp, tests/test_counter_state.cpp,
tests/test_memory_truth_gate.cpp).  Exit code 77 means "no GPU" as in MotifCL's CTest setup."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BUILD = os.path.join(ROOT, "motifcl_amd", "host", "build")
TESTS = ["test_counter_fused", "test_counter_state", "test_memory_gate", "test_layer_errors",
         "test_checkpoint", "test_adam", "test_deferred_updates"]


def _built():
    return all(os.path.exists(os.path.join(BUILD, t)) for t in TESTS)


def test_host_layer_is_built_and_skips_cleanly_without_a_gpu():
    if not _built():
        subprocess.run(["make", "-C", os.path.join(ROOT, "motifcl_amd", "host"), "-j8"], check=True,
                       capture_output=True)
    assert _built()
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present: the executables run for real in the gpu-marked test")
    r = subprocess.run([os.path.join(BUILD, "test_layer_errors")], capture_output=True, text=True, timeout=120)
    assert r.returncode == 77, r.stdout + r.stderr  # skipped, not crashed


@pytest.mark.gpu
@pytest.mark.parametrize("name", TESTS)
def test_host_cpp(name):
    exe = os.path.join(BUILD, name)
    assert os.path.exists(exe), "build motifcl_amd/host first (__graft_entry__.build())"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    print(r.stdout)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
