"""ctypes loader for the CPU oracle (oracle/counter_oracle.c).

TEST INFRASTRUCTURE ONLY.  Imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py; never by anything under motifcl_amd/.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libcounter_oracle.so")

_u8p = ctypes.POINTER(ctypes.c_uint8)
_i8p = ctypes.POINTER(ctypes.c_int8)
_f32p = ctypes.POINTER(ctypes.c_float)
_c_int, _c_float, _c_u32 = ctypes.c_int, ctypes.c_float, ctypes.c_uint32


def build():
    """Compile libcounter_oracle.so with gcc (recipe: oracle/Makefile)."""
    subprocess.run(["make", "-C", _HERE, "-B"], check=True, capture_output=True)


def _load():
    if not os.path.exists(_SO):
        build()
    lib = ctypes.CDLL(_SO)
    lib.oracle_hash_u32.restype = _c_u32
    lib.oracle_hash_u32.argtypes = [_c_u32]
    lib.oracle_uniform01.restype = _c_float
    lib.oracle_uniform01.argtypes = [_c_u32]
    lib.oracle_encode.restype = _c_int
    lib.oracle_encode.argtypes = [_c_int, _c_int, _c_int]
    lib.oracle_decode.restype = None
    lib.oracle_decode.argtypes = [_c_int, _c_int, ctypes.POINTER(_c_int), ctypes.POINTER(_c_int)]
    lib.oracle_tick_code.restype = _c_int
    lib.oracle_tick_code.argtypes = [_c_int, _c_float, _c_float, _c_float, _c_float,
                                     _c_int, _c_float, _c_u32, _c_u32]
    lib.oracle_pack_codes.restype = None
    lib.oracle_pack_codes.argtypes = [_u8p, ctypes.c_size_t, _u8p]
    lib.oracle_unpack_codes.restype = None
    lib.oracle_unpack_codes.argtypes = [_u8p, ctypes.c_size_t, _u8p]
    lib.oracle_decode_weight.restype = None
    lib.oracle_decode_weight.argtypes = [_u8p, _f32p, _f32p, _c_int, _c_int, _c_int]
    lib.oracle_row_stats.restype = None
    lib.oracle_row_stats.argtypes = [_u8p, _f32p, _f32p, _f32p, _f32p, _f32p,
                                     _c_int, _c_int, _c_int, _c_float, _c_float, _c_float]
    lib.oracle_apply_update.restype = None
    lib.oracle_apply_update.argtypes = [_u8p, _f32p, _f32p, _f32p, _f32p,
                                        _c_int, _c_int, _c_int, _c_float, _c_u32]
    lib.oracle_update_dense.restype = _c_int
    lib.oracle_update_dense.argtypes = [_u8p, _f32p, _f32p, _f32p, _c_int, _c_int, _c_int,
                                        _c_float, _c_float, _c_float, _c_float, _c_u32]
    lib.oracle_grad_w_seq.restype = None
    lib.oracle_grad_w_seq.argtypes = [_f32p, _f32p, _f32p, _c_int, _c_int, _c_int]
    lib.oracle_update_fused.restype = _c_int
    lib.oracle_update_fused.argtypes = [_u8p, _f32p, _f32p, _f32p, _f32p, _f32p,
                                        _c_int, _c_int, _c_int, _c_int,
                                        _c_float, _c_float, _c_float, _c_float, _c_u32]
    lib.oracle_forward.restype = None
    lib.oracle_forward.argtypes = [_f32p, _u8p, _f32p, _f32p, _c_int, _c_int, _c_int, _c_int]
    lib.oracle_backward_input.restype = None
    lib.oracle_backward_input.argtypes = [_f32p, _u8p, _f32p, _f32p, _c_int, _c_int, _c_int, _c_int]
    lib.oracle_init_state.restype = None
    lib.oracle_init_state.argtypes = [_i8p, _u8p, _f32p, _f32p, _c_int, _c_int, _c_int, _c_float]
    lib.oracle_sgd_update.restype = None
    lib.oracle_sgd_update.argtypes = [_f32p, _f32p, ctypes.c_size_t, _c_float]
    lib.oracle_adam_update.restype = None
    lib.oracle_adam_update.argtypes = [_f32p, _f32p, _f32p, _f32p, ctypes.c_size_t, _c_float, _c_float,
                                       _c_float, _c_float, _c_int, _c_float]
    lib.oracle_num_threads.restype = _c_int
    lib.oracle_set_num_threads.argtypes = [_c_int]
    return lib


_lib = _load()


def _u8(a):
    assert a.dtype == np.uint8 and a.flags.c_contiguous
    return a.ctypes.data_as(_u8p)


def _f32(a):
    assert a.dtype == np.float32 and a.flags.c_contiguous
    return a.ctypes.data_as(_f32p)


def hash_u32(x):
    return int(_lib.oracle_hash_u32(int(x) & 0xFFFFFFFF))


def uniform01(x):
    return float(_lib.oracle_uniform01(int(x) & 0xFFFFFFFF))


def encode(t, c, C):
    return int(_lib.oracle_encode(t, c, C))


def decode(code, C):
    t, c = _c_int(), _c_int()
    _lib.oracle_decode(code, C, ctypes.byref(t), ctypes.byref(c))
    return t.value, c.value


def tick_code(code, gw, s_old, s_new, dn, C, lr, seed, elem):
    return int(_lib.oracle_tick_code(code, gw, s_old, s_new, dn, C, lr,
                                     int(seed) & 0xFFFFFFFF, int(elem) & 0xFFFFFFFF))


def pack_codes(codes):
    """uint8 codes (len % 4 == 0, values < 64) -> packed state bytes (3 per 4 codes)."""
    codes = np.ascontiguousarray(codes, dtype=np.uint8).reshape(-1)
    assert codes.size % 4 == 0
    state = np.empty(codes.size // 4 * 3, dtype=np.uint8)
    _lib.oracle_pack_codes(_u8(codes), codes.size, _u8(state))
    return state


def unpack_codes(state):
    state = np.ascontiguousarray(state, dtype=np.uint8).reshape(-1)
    assert state.size % 3 == 0
    codes = np.empty(state.size // 3 * 4, dtype=np.uint8)
    _lib.oracle_unpack_codes(_u8(state), codes.size, _u8(codes))
    return codes


def decode_weight(state, scale, C, in_features, out_features):
    w = np.empty((out_features, in_features), dtype=np.float32)
    _lib.oracle_decode_weight(_u8(state), _f32(scale), _f32(w), C, in_features, out_features)
    return w


def row_stats(state, scale, v, grad_w, C, lr_scale, rms_beta, rms_eps):
    """Returns (v_new, scale_new, denom); inputs untouched."""
    out_features, in_features = grad_w.shape
    v_new = v.copy()
    scale_new = np.empty(out_features, dtype=np.float32)
    denom = np.empty(out_features, dtype=np.float32)
    _lib.oracle_row_stats(_u8(state), _f32(scale), _f32(v_new), _f32(grad_w), _f32(scale_new),
                          _f32(denom), C, in_features, out_features, lr_scale, rms_beta, rms_eps)
    return v_new, scale_new, denom


def update_dense(state, scale, v, grad_w, C, lr, lr_scale, rms_beta, rms_eps, seed):
    """apply_update_seed semantics.  Returns new (state, scale, v); inputs untouched."""
    out_features, in_features = grad_w.shape
    state, scale, v = state.copy(), scale.copy(), v.copy()
    rc = _lib.oracle_update_dense(_u8(state), _f32(scale), _f32(v), _f32(grad_w),
                                  C, in_features, out_features, lr, lr_scale, rms_beta, rms_eps,
                                  int(seed) & 0xFFFFFFFF)
    assert rc == 0
    return state, scale, v


def grad_w_seq(grad_out, x):
    N, out_features = grad_out.shape
    N2, in_features = x.shape
    assert N == N2
    g = np.empty((out_features, in_features), dtype=np.float32)
    _lib.oracle_grad_w_seq(_f32(grad_out), _f32(x), _f32(g), in_features, out_features, N)
    return g


def update_fused(state, scale, v, grad_out, x, C, lr, lr_scale, rms_beta, rms_eps, seed):
    """apply_update_backward semantics.  Returns new (state, scale, v, grad_w)."""
    N, out_features = grad_out.shape
    in_features = x.shape[1]
    state, scale, v = state.copy(), scale.copy(), v.copy()
    g = np.empty((out_features, in_features), dtype=np.float32)
    rc = _lib.oracle_update_fused(_u8(state), _f32(scale), _f32(v), _f32(grad_out), _f32(x), _f32(g),
                                  C, in_features, out_features, N, lr, lr_scale, rms_beta, rms_eps,
                                  int(seed) & 0xFFFFFFFF)
    assert rc == 0
    return state, scale, v, g


def forward(x, state, scale, C, out_features):
    N, in_features = x.shape
    y = np.empty((N, out_features), dtype=np.float32)
    _lib.oracle_forward(_f32(x), _u8(state), _f32(scale), _f32(y), C, in_features, out_features, N)
    return y


def backward_input(grad_out, state, scale, C, in_features):
    N, out_features = grad_out.shape
    gx = np.empty((N, in_features), dtype=np.float32)
    _lib.oracle_backward_input(_f32(grad_out), _u8(state), _f32(scale), _f32(gx),
                               C, in_features, out_features, N)
    return gx


def init_state(tern, C, init_gain=1.0):
    """tern int8 [out,in] in {-1,0,1} -> (state, scale, v) as the layer constructor packs them."""
    tern = np.ascontiguousarray(tern, dtype=np.int8)
    out_features, in_features = tern.shape
    state = np.empty(out_features * (in_features // 4) * 3, dtype=np.uint8)
    scale = np.empty(out_features, dtype=np.float32)
    v = np.empty(out_features, dtype=np.float32)
    _lib.oracle_init_state(tern.ctypes.data_as(_i8p), _u8(state), _f32(scale), _f32(v),
                           C, in_features, out_features, init_gain)
    return state, scale, v


def sgd_update(param, grad, lr):
    """Returns the updated parameter (kernels/optim.cl:1-7)."""
    p = np.array(param, dtype=np.float32, copy=True).reshape(-1)
    g = np.ascontiguousarray(grad, dtype=np.float32).reshape(-1)
    _lib.oracle_sgd_update(_f32(p), _f32(g), p.size, lr)
    return p.reshape(np.shape(param))


def adam_update(param, grad, m, v, lr, beta1, beta2, eps, step, weight_decay=0.0):
    """Returns (param, m, v) after one Adam step (kernels/optim.cl:31-53, src/ops/optim.cpp:65-86)."""
    p, mm, vv = (np.array(a, dtype=np.float32, copy=True).reshape(-1) for a in (param, m, v))
    g = np.ascontiguousarray(grad, dtype=np.float32).reshape(-1)
    _lib.oracle_adam_update(_f32(p), _f32(g), _f32(mm), _f32(vv), p.size, lr, beta1, beta2, eps, step,
                            weight_decay)
    shape = np.shape(param)
    return p.reshape(shape), mm.reshape(shape), vv.reshape(shape)


def num_threads():
    return int(_lib.oracle_num_threads())


def set_num_threads(n):
    _lib.oracle_set_num_threads(int(n))
