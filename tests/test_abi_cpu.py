"""CPU-only checks of the C-ABI library: it loads, exports every declared symbol, and
rejects invalid arguments before touching the GPU (no compute calls are made here).
Validation cases follow src/runtime/vulkan_backend.cpp:8497-8521 and
tests/test_vulkan_runtime_standalone.cpp:19-23 (in_features = 3 is rejected)."""
import ctypes
import os
import re

import pytest

import motifcl_amd
from motifcl_amd import lib as mlib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
P = 0x1000  # fake non-null device address; validation must fail before it is ever used
INF, NAN = float("inf"), float("nan")


@pytest.fixture(scope="module")
def L():
    return motifcl_amd.load()


def test_every_declared_symbol_is_exported_and_bound(L):
    for header_name, table in (("motifcl_amd.h", mlib.SIGNATURES), ("motifcl_amd_diag.h", mlib.DIAG_SIGNATURES)):
        header = open(os.path.join(ROOT, "include", header_name)).read()
        declared = set(re.findall(r"\b(mcc_[a-z0-9_]+)\s*\(", header))
        assert declared == set(table), declared ^ set(table)
        for name in declared:
            assert hasattr(L, name)


def _dense(L, C=11, n_in=8, n_out=2, lr=3e-3, lr_scale=0.0, beta=0.9, eps=1e-3,
           state_n=None, row_n=None, g_n=None):
    groups = n_out * (n_in // 4) if n_in else 0
    return L.mcc_compact_counter_apply_update_dense(
        None, P, groups * 3 if state_n is None else state_n,
        P, n_out * 4 if row_n is None else row_n, P, n_out * 4 if row_n is None else row_n,
        P, n_out * n_in * 4 if g_n is None else g_n, C, n_in, n_out, lr, lr_scale, beta, eps, 1)


@pytest.mark.parametrize("kwargs,needle", [
    (dict(n_in=0), "non-zero"),
    (dict(n_out=0), "non-zero"),
    (dict(n_in=6), "divisible by 4"),
    (dict(C=0), "6-bit"),
    (dict(C=12), "6-bit"),
    (dict(lr=NAN), "finite lr"),
    (dict(lr=INF), "finite lr"),
    (dict(lr_scale=NAN), "finite lr_scale"),
    (dict(beta=INF), "finite rms_beta"),
    (dict(eps=-1.0), "non-negative finite rms_eps"),
    (dict(eps=NAN), "non-negative finite rms_eps"),
    (dict(state_n=11), "state buffer is too small"),
    (dict(row_n=4), "per-row buffer is too small"),
    (dict(g_n=60), "gradient buffer is too small"),
])
def test_dense_update_rejects(L, kwargs, needle):
    rc = _dense(L, **kwargs)
    assert rc == -1
    assert needle in L.mcc_last_error().decode()


def test_fused_update_rejects(L):
    def fused(batch=2, n_in=8, n_out=2, C=3, ws=None, x_n=None, lr=0.05):
        return L.mcc_compact_counter_apply_update_fused(
            None, P, n_out * (n_in // 4) * 3, P, n_out * 4, P, n_out * 4,
            P, batch * n_out * 4, P, batch * n_in * 4 if x_n is None else x_n,
            P, n_out * n_in * 4 if ws is None else ws,
            C, n_in, n_out, batch, lr, 0.01, 0.9, 1e-8, 777)
    assert fused(batch=0) == -1 and "non-zero" in L.mcc_last_error().decode()
    assert fused(n_in=3) == -1 and "divisible by 4" in L.mcc_last_error().decode()
    assert fused(ws=8) == -1 and "workspace is too small" in L.mcc_last_error().decode()
    assert fused(x_n=8) == -1 and "activation buffer is too small" in L.mcc_last_error().decode()
    assert fused(lr=NAN) == -1 and "finite lr" in L.mcc_last_error().decode()
    assert L.mcc_compact_counter_fused_workspace_nbytes(8, 2, 2) == 64
    assert L.mcc_compact_counter_fused_workspace_nbytes(0, 2, 2) == 0


def test_linear_entry_points_reject(L):
    # in_features = 3 (tests/test_vulkan_runtime_standalone.cpp:19-23)
    rc = L.mcc_compact_counter_backward_input_u8(None, P, 3, P, 4, P, 4, P, 12, 1, 3, 1, 3)
    assert rc == -1 and L.mcc_last_error().decode() != ""
    rc = L.mcc_compact_counter_decode_weight(None, P, 2, P, 8, P, 32, 4, 2, 3)
    assert rc == -1 and "state buffer is too small" in L.mcc_last_error().decode()
    rc = L.mcc_compact_counter_forward_u8(None, P, 32, P, 6, P, 8, P, 4, 2, 4, 2, 3)
    assert rc == -1 and "activation buffer is too small" in L.mcc_last_error().decode()
    rc = L.mcc_compact_counter_forward_u8(None, P, 32, P, 6, P, 8, P, 16, 2, 4, 2, 40)
    assert rc == -1 and "6-bit" in L.mcc_last_error().decode()
    rc = L.mcc_matmul_transpose_a_f32(None, P, 4, P, 4, P, 4, 0, 1, 1)
    assert rc == -1 and "non-zero" in L.mcc_last_error().decode()
    rc = L.mcc_matmul_transpose_a_f32(None, P, 4, P, 4, P, 4, 2, 1, 1)
    assert rc == -1 and "too small" in L.mcc_last_error().decode()


def test_storage_rejects_without_touching_the_device(L):
    p = ctypes.c_void_p()
    assert L.mcc_device_alloc(ctypes.byref(p), 0) == -1
    assert "zero-byte" in L.mcc_last_error().decode()
    assert L.mcc_device_free(None) == 0
    assert L.mcc_device_free(P) == -1
    assert L.mcc_device_bytes_current() == 0


def _counter_tensor(state_ptr, n_in=8, n_out=2):
    t = mlib.CounterTensor()
    t.state, t.state_nbytes = state_ptr, n_out * (n_in // 4) * 3
    t.scale, t.scale_nbytes, t.v, t.v_nbytes = P, n_out * 4, P, n_out * 4
    t.grad_w, t.grad_w_nbytes = P, n_out * n_in * 4
    t.in_features, t.out_features, t.lr, t.seed = n_in, n_out, 3e-3, 1
    return t


def test_batched_updates_reject_a_state_listed_twice_and_validate_every_tensor_first(L):
    # two descriptors on one state would be updated by two sets of workgroups of the same launch
    arr = (mlib.CounterTensor * 3)(_counter_tensor(0x1000), _counter_tensor(0x2000), _counter_tensor(0x1000))
    assert L.mcc_compact_counter_apply_update_dense_batched(None, arr, 3, 11, 0.0, 0.9, 1e-3) == -1
    assert "same state twice" in L.mcc_last_error().decode()
    # an invalid tensor anywhere in the list is reported before anything is enqueued
    arr = (mlib.CounterTensor * 2)(_counter_tensor(0x1000), _counter_tensor(0x2000, n_in=6))
    assert L.mcc_compact_counter_apply_update_dense_batched(None, arr, 2, 11, 0.0, 0.9, 1e-3) == -1
    assert L.mcc_last_error().decode().startswith("tensor 1:")

    def fused(state_ptr, n_in=8):
        t = mlib.FusedTensor()
        t.state, t.state_nbytes = state_ptr, 2 * (n_in // 4) * 3
        t.scale, t.scale_nbytes, t.v, t.v_nbytes = P, 8, P, 8
        t.grad_out, t.grad_out_nbytes, t.x, t.x_nbytes = P, 4 * 2 * 4, P, 4 * n_in * 4
        t.in_features, t.out_features, t.batch, t.lr, t.seed = n_in, 2, 4, 3e-3, 1
        return t

    for mode in (0, 1):  # fp32 instruction, split-bf16 contraction: the same checks before any launch
        assert L.mcc_set_contraction_mode(mode) == 0
        try:
            arr = (mlib.FusedTensor * 2)(fused(0x1000), fused(0x1000))
            need = L.mcc_compact_counter_fused_batched_workspace_nbytes(arr, 2)
            assert L.mcc_compact_counter_apply_update_fused_batched(None, arr, 2, 0x10000, need, 11, 0.0, 0.9, 1e-3) == -1
            assert "same state twice" in L.mcc_last_error().decode()
            arr = (mlib.FusedTensor * 2)(fused(0x1000), fused(0x2000, n_in=6))
            need = L.mcc_compact_counter_fused_batched_workspace_nbytes(arr, 2)
            assert L.mcc_compact_counter_apply_update_fused_batched(None, arr, 2, 0x10000, need, 11, 0.0, 0.9, 1e-3) == -1
            assert L.mcc_last_error().decode().startswith("tensor 1:")
        finally:
            L.mcc_set_contraction_mode(0)


def test_package_fails_loudly_without_the_library():
    # no CPU path stands in for the HIP library: with the shared object missing, loading raises
    import subprocess
    import sys
    code = (
        "import motifcl_amd\n"
        "from motifcl_amd.lib import LibraryMissing\n"
        "try:\n"
        "    motifcl_amd.load()\n"
        "except LibraryMissing as e:\n"
        "    print('missing:', e)\n"
        "else:\n"
        "    raise SystemExit('loaded something')\n"
        "from motifcl_amd import ops\n"
        "try:\n"
        "    ops.fused_workspace_nbytes(8, 8, 8)\n"
        "except LibraryMissing:\n"
        "    print('op raised')\n"
        "else:\n"
        "    raise SystemExit('op answered without the library')\n"
    )
    env = dict(os.environ, MOTIFCL_AMD_LIB="/nonexistent/libmotifcl_amd.so")
    out = subprocess.run([sys.executable, "-c", code], cwd=ROOT, env=env, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "missing:" in out.stdout and "op raised" in out.stdout
