"""Thin Python front of the C ABI.  torch is used only as the owner of device
memory and of the current HIP stream; every computation happens in
libmotifcl_amd.so."""
import ctypes

import torch

from . import lib as _lib


def _stream():
    return torch.cuda.current_stream().cuda_stream or None


def _buf(t, dtype):
    if not t.is_cuda:
        raise ValueError("expected a device tensor")
    if t.dtype != dtype:
        raise ValueError("expected dtype %s, got %s" % (dtype, t.dtype))
    if not t.is_contiguous():
        raise ValueError("expected a contiguous tensor")
    return t.data_ptr(), t.numel() * t.element_size()


def apply_update_dense(state, scale, v, grad_w, C, lr, lr_scale, rms_beta, rms_eps, seed,
                       in_features=None, out_features=None):
    """In-place update-only step (CounterStateLinear::apply_update_seed)."""
    L = _lib.load()
    if in_features is None:
        out_features, in_features = grad_w.shape
    _lib.check(L.mcc_compact_counter_apply_update_dense(
        _stream(), *_buf(state, torch.uint8), *_buf(scale, torch.float32), *_buf(v, torch.float32),
        *_buf(grad_w, torch.float32), C, in_features, out_features,
        lr, lr_scale, rms_beta, rms_eps, seed & 0xFFFFFFFF))


class UpdateBatch:
    """A reusable descriptor list for apply_update_dense_batched: tensors are
    (state, scale, v, grad_w) device tensors with grad_w of shape [out, in]."""

    def __init__(self, tensors, lr, seeds):
        self._keep = list(tensors)
        n = len(self._keep)
        self.array = (_lib.CounterTensor * n)()
        for i, (state, scale, v, grad_w) in enumerate(self._keep):
            out_features, in_features = grad_w.shape
            d = self.array[i]
            d.state, d.state_nbytes = _buf(state, torch.uint8)
            d.scale, d.scale_nbytes = _buf(scale, torch.float32)
            d.v, d.v_nbytes = _buf(v, torch.float32)
            d.grad_w, d.grad_w_nbytes = _buf(grad_w, torch.float32)
            d.in_features, d.out_features = in_features, out_features
            d.lr = lr[i] if isinstance(lr, (list, tuple)) else lr
            d.seed = seeds[i] & 0xFFFFFFFF
        self.n = n

    def set_seeds(self, seeds):
        for i in range(self.n):
            self.array[i].seed = seeds[i] & 0xFFFFFFFF


def apply_update_dense_batched(batch, C, lr_scale, rms_beta, rms_eps):
    """In-place update-only step of every tensor of an UpdateBatch, one call."""
    L = _lib.load()
    _lib.check(L.mcc_compact_counter_apply_update_dense_batched(
        _stream(), batch.array, batch.n, C, lr_scale, rms_beta, rms_eps))


class FusedBatch:
    """A reusable descriptor list for apply_update_fused_batched: tensors are
    (state, scale, v, grad_out [batch, out], x [batch, in]) device tensors."""

    def __init__(self, tensors, lr, seeds):
        self._keep = list(tensors)
        n = len(self._keep)
        self.array = (_lib.FusedTensor * n)()
        for i, (state, scale, v, grad_out, x) in enumerate(self._keep):
            batch, out_features = grad_out.shape
            d = self.array[i]
            d.state, d.state_nbytes = _buf(state, torch.uint8)
            d.scale, d.scale_nbytes = _buf(scale, torch.float32)
            d.v, d.v_nbytes = _buf(v, torch.float32)
            d.grad_out, d.grad_out_nbytes = _buf(grad_out, torch.float32)
            d.x, d.x_nbytes = _buf(x, torch.float32)
            d.in_features, d.out_features, d.batch = x.shape[1], out_features, batch
            d.lr = lr[i] if isinstance(lr, (list, tuple)) else lr
            d.seed = seeds[i] & 0xFFFFFFFF
        self.n = n

    def set_seeds(self, seeds):
        for i in range(self.n):
            self.array[i].seed = seeds[i] & 0xFFFFFFFF

    def workspace_nbytes(self):
        return int(_lib.load().mcc_compact_counter_fused_batched_workspace_nbytes(self.array, self.n))


def apply_update_fused_batched(batch, workspace, C, lr_scale, rms_beta, rms_eps):
    """In-place fused step of every tensor of a FusedBatch in a handful of launches."""
    L = _lib.load()
    _lib.check(L.mcc_compact_counter_apply_update_fused_batched(
        _stream(), batch.array, batch.n, *_buf(workspace, torch.uint8), C, lr_scale, rms_beta, rms_eps))


def fused_workspace_nbytes(in_features, out_features, batch):
    return int(_lib.load().mcc_compact_counter_fused_workspace_nbytes(in_features, out_features, batch))


def fused_strip_workspace_nbytes(in_features, out_features, batch):
    """Size of the small workspace of the accumulator-resident fused step; 0 if unsupported."""
    return int(_lib.load().mcc_compact_counter_fused_strip_workspace_nbytes(in_features, out_features, batch))


def fused_check(workspace, in_features, out_features, batch):
    """Waits for the stream and raises MccError if a strip-workspace step gave up a wait."""
    L = _lib.load()
    ptr, nbytes = (0, 0) if workspace is None else (workspace.data_ptr(), workspace.numel() * workspace.element_size())
    _lib.check(L.mcc_compact_counter_fused_check(_stream(), ptr, nbytes, in_features, out_features, batch))


def apply_update_fused(state, scale, v, grad_out, x, workspace, C, lr, lr_scale, rms_beta, rms_eps,
                       seed):
    """In-place fused step (CounterStateLinear::apply_update_backward)."""
    L = _lib.load()
    batch, out_features = grad_out.shape
    in_features = x.shape[1]
    if x.shape[0] != batch:
        raise ValueError("x and grad_out disagree on the batch size")
    _lib.check(L.mcc_compact_counter_apply_update_fused(
        _stream(), *_buf(state, torch.uint8), *_buf(scale, torch.float32), *_buf(v, torch.float32),
        *_buf(grad_out, torch.float32), *_buf(x, torch.float32),
        workspace.data_ptr(), workspace.numel() * workspace.element_size(),
        C, in_features, out_features, batch, lr, lr_scale, rms_beta, rms_eps, seed & 0xFFFFFFFF))


NOALLOC_WORKSPACE_NBYTES = 32 << 20  # MCC_NOALLOC_WORKSPACE_NBYTES of include/motifcl_amd.h


def apply_update_fused_static(state, scale, v, grad_out, x, C, lr, lr_scale, rms_beta, rms_eps, seed):
    """The fused step on the library's own static workspace: the call allocates nothing."""
    L = _lib.load()
    batch, out_features = grad_out.shape
    in_features = x.shape[1]
    if x.shape[0] != batch:
        raise ValueError("x and grad_out disagree on the batch size")
    _lib.check(L.mcc_compact_counter_apply_update_fused_static(
        _stream(), *_buf(state, torch.uint8), *_buf(scale, torch.float32), *_buf(v, torch.float32),
        *_buf(grad_out, torch.float32), *_buf(x, torch.float32),
        C, in_features, out_features, batch, lr, lr_scale, rms_beta, rms_eps, seed & 0xFFFFFFFF))


def matmul_transpose_a(a, b, out=None):
    """c[m,n] = a[k,m]^T . b[k,n]."""
    L = _lib.load()
    k, m = a.shape
    k2, n = b.shape
    if k != k2:
        raise ValueError("matmul_transpose_a: leading dimensions differ")
    if out is None:
        out = torch.empty((m, n), dtype=torch.float32, device=a.device)
    _lib.check(L.mcc_matmul_transpose_a_f32(_stream(), *_buf(a, torch.float32), *_buf(b, torch.float32),
                                            *_buf(out, torch.float32), k, m, n))
    return out


def decode_weight(state, scale, C, in_features, out_features, out=None):
    L = _lib.load()
    w = out if out is not None else torch.empty((out_features, in_features), dtype=torch.float32, device=state.device)
    _lib.check(L.mcc_compact_counter_decode_weight(
        _stream(), *_buf(state, torch.uint8), *_buf(scale, torch.float32), *_buf(w, torch.float32),
        in_features, out_features, C))
    return w


def forward(x, state, scale, C, out_features, out=None):
    L = _lib.load()
    batch, in_features = x.shape
    y = out if out is not None else torch.empty((batch, out_features), dtype=torch.float32, device=x.device)
    _lib.check(L.mcc_compact_counter_forward_u8(
        _stream(), *_buf(x, torch.float32), *_buf(state, torch.uint8), *_buf(scale, torch.float32),
        *_buf(y, torch.float32), batch, in_features, out_features, C))
    return y


def backward_input(grad_out, state, scale, C, in_features, out=None):
    L = _lib.load()
    batch, out_features = grad_out.shape
    gx = out if out is not None else torch.empty((batch, in_features), dtype=torch.float32, device=grad_out.device)
    _lib.check(L.mcc_compact_counter_backward_input_u8(
        _stream(), *_buf(state, torch.uint8), *_buf(scale, torch.float32),
        *_buf(grad_out, torch.float32), *_buf(gx, torch.float32),
        batch, in_features, out_features, C))
    return gx


def sgd_update(param, grad, lr):
    """param -= lr * grad in place (sgd_update of MotifCL)."""
    L = _lib.load()
    _lib.check(L.mcc_sgd_update_f32(_stream(), *_buf(param, torch.float32), *_buf(grad, torch.float32),
                                    param.numel(), lr))


def adam_update(param, grad, m, v, lr, beta1, beta2, eps, step, weight_decay=0.0):
    """In-place Adam step with decoupled weight decay (adam_update_fast of MotifCL)."""
    L = _lib.load()
    _lib.check(L.mcc_adam_update_f32(_stream(), *_buf(param, torch.float32), *_buf(grad, torch.float32),
                                     *_buf(m, torch.float32), *_buf(v, torch.float32), param.numel(),
                                     lr, beta1, beta2, eps, step, weight_decay))


CONTRACTION_FP32, CONTRACTION_BF16X6 = 0, 1


def set_contraction_mode(mode):
    """Process-wide choice of the weight-gradient contraction: fp32 matrix instruction or split bf16."""
    _lib.check(_lib.load().mcc_set_contraction_mode(int(mode)))


def get_contraction_mode():
    return int(_lib.load().mcc_get_contraction_mode())


def fill_normal(t, stream_id, sigma):
    """t[i] = sigma * z_i from the library's counter-based generator (lowbias32 -> Box-Muller)."""
    ptr, nbytes = _buf(t, torch.float32)
    _lib.check(_lib.load().mcc_fill_normal_f32(_stream(), ptr, nbytes // 4, stream_id & 0xFFFFFFFF, sigma))
    return t


def fill_counter_state(state, stream_id, n_codes):
    """Packed state with every code uniform on [0, n_codes), same generator."""
    ptr, nbytes = _buf(state, torch.uint8)
    if nbytes % 3:
        raise ValueError("a packed state holds 3 bytes per group")
    _lib.check(_lib.load().mcc_fill_counter_state_u8(_stream(), ptr, nbytes // 3, stream_id & 0xFFFFFFFF, n_codes))
    return state


class ClockProbe:
    """Shader clock while other kernels run: a one-wave kernel on a side stream sleeps for
    `seconds` of the constant-rate wall clock and counts shader cycles over the same stretch.

        probe = ClockProbe(0.05)      # starts now, on its own stream
        ... launch the kernels under test on the current stream ...
        torch.cuda.synchronize()
        mhz = probe.mhz()
    """

    def __init__(self, seconds):
        L = _lib.load()
        khz = ctypes.c_int(0)
        _lib.check(L.mcc_wall_clock_khz(ctypes.byref(khz)))
        self._khz = khz.value
        self._out = torch.zeros(2, dtype=torch.int64, device="cuda")
        self._stream = torch.cuda.Stream()
        torch.cuda.synchronize()
        _lib.check(L.mcc_clock_probe(ctypes.c_void_p(self._stream.cuda_stream), ctypes.c_void_p(self._out.data_ptr()),
                                     16, float(seconds)))

    def mhz(self):
        self._stream.synchronize()
        wall, cycles = (int(v) for v in self._out.tolist())
        if wall <= 0:
            raise RuntimeError("clock probe has not run")
        return cycles / wall * self._khz / 1000.0
