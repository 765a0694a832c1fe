"""Loads libmotifcl_amd.so and declares the C ABI of include/motifcl_amd.h for ctypes."""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("MOTIFCL_AMD_LIB", os.path.join(HERE, "libmotifcl_amd.so"))

_vp, _sz, _f, _u32 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_float, ctypes.c_uint32

# name -> (restype, argtypes); one entry per declaration in include/motifcl_amd.h
SIGNATURES = {
    "mcc_last_error": (ctypes.c_char_p, []),
    "mcc_device_name": (ctypes.c_char_p, []),
    "mcc_compact_counter_apply_update_dense": (
        ctypes.c_int, [_vp, _vp, _sz, _vp, _sz, _vp, _sz, _vp, _sz, _sz, _sz, _sz, _f, _f, _f, _f, _u32]),
    "mcc_compact_counter_apply_update_dense_batched": (
        ctypes.c_int, [_vp, _vp, _sz, _sz, _f, _f, _f]),
    "mcc_compact_counter_fused_workspace_nbytes": (_sz, [_sz, _sz, _sz]),
    "mcc_compact_counter_fused_strip_workspace_nbytes": (_sz, [_sz, _sz, _sz]),
    "mcc_compact_counter_fused_check": (ctypes.c_int, [_vp, _vp, _sz, _sz, _sz, _sz]),
    "mcc_compact_counter_apply_update_fused": (
        ctypes.c_int, [_vp, _vp, _sz, _vp, _sz, _vp, _sz, _vp, _sz, _vp, _sz, _vp, _sz,
                       _sz, _sz, _sz, _sz, _f, _f, _f, _f, _u32]),
    "mcc_compact_counter_apply_update_fused_static": (
        ctypes.c_int, [_vp, _vp, _sz, _vp, _sz, _vp, _sz, _vp, _sz, _vp, _sz,
                       _sz, _sz, _sz, _sz, _f, _f, _f, _f, _u32]),
    "mcc_compact_counter_fused_batched_workspace_nbytes": (_sz, [_vp, _sz]),
    "mcc_compact_counter_apply_update_fused_batched": (
        ctypes.c_int, [_vp, _vp, _sz, _vp, _sz, _sz, _f, _f, _f]),
    "mcc_set_contraction_mode": (ctypes.c_int, [ctypes.c_int]),
    "mcc_get_contraction_mode": (ctypes.c_int, []),
    "mcc_matmul_transpose_a_f32": (ctypes.c_int, [_vp, _vp, _sz, _vp, _sz, _vp, _sz, _sz, _sz, _sz]),
    "mcc_compact_counter_decode_weight": (ctypes.c_int, [_vp, _vp, _sz, _vp, _sz, _vp, _sz, _sz, _sz, _sz]),
    "mcc_compact_counter_forward_u8": (
        ctypes.c_int, [_vp, _vp, _sz, _vp, _sz, _vp, _sz, _vp, _sz, _sz, _sz, _sz, _sz]),
    "mcc_compact_counter_backward_input_u8": (
        ctypes.c_int, [_vp, _vp, _sz, _vp, _sz, _vp, _sz, _vp, _sz, _sz, _sz, _sz, _sz]),
    "mcc_sgd_update_f32": (ctypes.c_int, [_vp, _vp, _sz, _vp, _sz, _sz, _f]),
    "mcc_adam_update_f32": (ctypes.c_int, [_vp, _vp, _sz, _vp, _sz, _vp, _sz, _vp, _sz, _sz, _f, _f, _f, _f,
                                           ctypes.c_int, _f]),
    "mcc_device_alloc": (ctypes.c_int, [ctypes.POINTER(_vp), _sz]),
    "mcc_device_free": (ctypes.c_int, [_vp]),
    "mcc_device_pool_clear": (ctypes.c_int, []),
    "mcc_device_bytes_current": (_sz, []),
    "mcc_device_bytes_peak": (_sz, []),
    "mcc_device_bytes_reset_peak": (None, []),
    "mcc_memcpy_h2d": (ctypes.c_int, [_vp, _vp, _vp, _sz]),
    "mcc_memcpy_d2h": (ctypes.c_int, [_vp, _vp, _vp, _sz]),
    "mcc_memset_zero": (ctypes.c_int, [_vp, _vp, _sz]),
    "mcc_stream_synchronize": (ctypes.c_int, [_vp]),
    "mcc_profiler_enable": (None, [ctypes.c_int]),
    "mcc_profiler_reset": (None, []),
    "mcc_profiler_query": (ctypes.c_int, [ctypes.c_char_p, ctypes.POINTER(ctypes.c_double),
                                          ctypes.POINTER(ctypes.c_uint64)]),
}

# measurement and test aids: one entry per declaration in include/motifcl_amd_diag.h
DIAG_SIGNATURES = {
    "mcc_compact_counter_fused_strip_set_spin_limit": (None, [ctypes.c_uint]),
    "mcc_compact_counter_fused_strip_set_tile_mode": (None, [ctypes.c_int, ctypes.c_int]),
    "mcc_compact_counter_fused_strip_workspace_nbytes_for_grid": (ctypes.c_size_t, [ctypes.c_size_t, ctypes.c_size_t,
                                                                                    ctypes.c_size_t, ctypes.c_int]),
    "mcc_contraction_spans_set_test_mode": (None, [ctypes.c_uint, ctypes.c_int]),
    "mcc_clock_probe": (ctypes.c_int, [_vp, _vp, _sz, ctypes.c_double]),
    "mcc_wall_clock_khz": (ctypes.c_int, [ctypes.POINTER(ctypes.c_int)]),
    "mcc_fill_normal_f32": (ctypes.c_int, [_vp, _vp, _sz, _u32, _f]),
    "mcc_fill_counter_state_u8": (ctypes.c_int, [_vp, _vp, _sz, _u32, _u32]),
}


class CounterTensor(ctypes.Structure):
    """struct mcc_counter_tensor of include/motifcl_amd.h."""
    _fields_ = [("state", _vp), ("state_nbytes", _sz), ("scale", _vp), ("scale_nbytes", _sz),
                ("v", _vp), ("v_nbytes", _sz), ("grad_w", _vp), ("grad_w_nbytes", _sz),
                ("in_features", _sz), ("out_features", _sz), ("lr", _f), ("seed", _u32)]


class FusedTensor(ctypes.Structure):
    """struct mcc_fused_tensor of include/motifcl_amd.h."""
    _fields_ = [("state", _vp), ("state_nbytes", _sz), ("scale", _vp), ("scale_nbytes", _sz),
                ("v", _vp), ("v_nbytes", _sz), ("grad_out", _vp), ("grad_out_nbytes", _sz),
                ("x", _vp), ("x_nbytes", _sz), ("in_features", _sz), ("out_features", _sz),
                ("batch", _sz), ("lr", _f), ("seed", _u32)]


_lib = None


class LibraryMissing(RuntimeError):
    pass


def load():
    """Returns the loaded library; raises LibraryMissing if it has not been built.

    There is no fallback path: without the HIP library nothing in this package computes."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise LibraryMissing(
            "%s is missing: build it with `python -m motifcl_amd.build` "
            "(or __graft_entry__.build())" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in list(SIGNATURES.items()) + list(DIAG_SIGNATURES.items()):
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


class MccError(RuntimeError):
    """Raised when a C-ABI call reports failure; carries mcc_last_error()."""

    def __init__(self, code, message):
        super().__init__("motifcl_amd error %d: %s" % (code, message))
        self.code = code
        self.message = message


def check(rc):
    if rc != 0:
        raise MccError(rc, load().mcc_last_error().decode())
