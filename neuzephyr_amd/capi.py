"""ctypes view of the C-ABI in include/nzhip.h (test and benchmark plumbing).

No fallback of any kind lives here: if libnzhip.so is missing or a call fails, an exception
is raised.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

ACT_NONE, ACT_RELU = 0, 1
LAYOUT_ROW, LAYOUT_TRANS = 0, 1

EXPORTS = [
    "nzhip_version", "nzhip_last_error", "nzhip_device_info", "nzhip_gemm", "nzhip_gemm_static",
    "nzhip_static_scratch_bytes", "nzhip_gemm_force_tile", "nzhip_gemm_coop_timeouts", "nzhip_gemm_coop_reset", "nzhip_gemm_coop_test_mode", "nzhip_probe_mfma", "nzhip_probe_copy", "nzhip_prepared_create", "nzhip_prepared_invalidate", "nzhip_prepared_fills",
    "nzhip_prepared_destroy", "nzhip_gemm_prepared_b", "nzhip_conv2d_forward_prepared", "nzhip_tensorcore_gemm",
    "nzhip_im2col", "nzhip_col2im", "nzhip_conv2d_forward", "nzhip_add_broadcast", "nzhip_relu", "nzhip_fill",
    "nzhip_gemm_backward", "nzhip_matmul_backward", "nzhip_relu_backward", "nzhip_add_backward",
    "nzhip_im2col_backward", "nzhip_col2im_backward", "nzhip_conv2d_backward_data", "nzhip_conv2d_backward_weights", "nzhip_conv2d_backward_bias", "nzhip_conv2d_backward_relu_bias", "nzhip_matmul_f32", "nzhip_sgd_step", "nzhip_adam_step", "nzhip_fill_many", "nzhip_sgd_step_many", "nzhip_adam_step_many",
    "nzhip_softmax", "nzhip_softmax_jacobian", "nzhip_softmax_backward",
    "nzhip_avgpool2d", "nzhip_avgpool2d_backward", "nzhip_avgpool2d_backward_overwrite", "nzhip_bce_loss", "nzhip_bce_backward", "nzhip_mse_loss", "nzhip_mse_backward", "nzhip_expand", "nzhip_compress",
    "nzhip_default_stream", "nzhip_malloc", "nzhip_free_async", "nzhip_free", "nzhip_host_malloc", "nzhip_host_free", "nzhip_memset",
    "nzhip_memcpy_h2d", "nzhip_memcpy_d2d", "nzhip_memcpy_d2h", "nzhip_sync_ptr", "nzhip_stream_wait", "nzhip_sync_all",
    "nzhip_allocator_stats", "nzhip_allocator_trim",
]


class NzHipError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"nzhip status {status}: {message}")
        self.status = status
        self.message = message


class GemmDesc(C.Structure):
    _fields_ = [
        ("A", C.c_void_p), ("B", C.c_void_p), ("C", C.c_void_p),
        ("M", C.c_int64), ("N", C.c_int64), ("K", C.c_int64),
        ("lda", C.c_int64), ("ldb", C.c_int64), ("ldc", C.c_int64),
        ("a_layout", C.c_int32), ("b_layout", C.c_int32),
        ("batch_n", C.c_int64), ("batch_c", C.c_int64),
        ("a_stride_n", C.c_int64), ("a_stride_c", C.c_int64),
        ("b_stride_n", C.c_int64), ("b_stride_c", C.c_int64),
        ("c_stride_n", C.c_int64), ("c_stride_c", C.c_int64),
        ("bias", C.c_void_p),
        ("bias_stride_row", C.c_int64), ("bias_stride_col", C.c_int64),
        ("bias_stride_n", C.c_int64), ("bias_stride_c", C.c_int64),
        ("activation", C.c_int32), ("reserved", C.c_int32),
    ]


def lib_path() -> str:
    return os.path.join(HERE, "libnzhip.so")


def load() -> C.CDLL:
    """Load libnzhip.so (built in-tree by neuzephyr_amd/build.py). Raises if it is absent."""
    global _LIB
    if _LIB is not None:
        return _LIB
    path = lib_path()
    if not os.path.exists(path):
        raise FileNotFoundError(f"{path} is not built; run `python -c 'import __graft_entry__ as g; g.build()'`")
    lib = C.CDLL(path)
    sz, vp, i64 = C.c_size_t, C.c_void_p, C.c_int64
    shape = C.c_size_t * 4
    lib.nzhip_version.restype = C.c_int
    lib.nzhip_last_error.restype = C.c_char_p
    lib.nzhip_device_info.argtypes = [C.POINTER(C.c_int), C.POINTER(sz), C.c_char_p, sz]
    lib.nzhip_gemm.argtypes = [C.POINTER(GemmDesc), vp]
    lib.nzhip_gemm_static.argtypes = [C.POINTER(GemmDesc), vp]
    lib.nzhip_static_scratch_bytes.restype = sz
    lib.nzhip_gemm_force_tile.argtypes = [C.POINTER(GemmDesc), C.c_int, vp]
    lib.nzhip_gemm_coop_timeouts.argtypes = [C.POINTER(C.c_uint)]
    lib.nzhip_gemm_coop_reset.argtypes = [C.c_uint]
    lib.nzhip_gemm_coop_test_mode.argtypes = [C.c_uint, C.c_int]
    lib.nzhip_probe_mfma.argtypes = [C.c_int, C.c_int, vp, sz, vp]
    lib.nzhip_probe_copy.argtypes = [vp, vp, sz, vp]
    lib.nzhip_prepared_create.argtypes = [C.POINTER(vp)]
    lib.nzhip_prepared_invalidate.argtypes = [vp]
    lib.nzhip_prepared_fills.argtypes = [vp, C.POINTER(C.c_ulonglong)]
    lib.nzhip_prepared_destroy.argtypes = [vp]
    lib.nzhip_gemm_prepared_b.argtypes = [C.POINTER(GemmDesc), vp, vp]
    lib.nzhip_conv2d_forward_prepared.argtypes = [vp, vp, vp, vp] + [sz] * 10 + [i64, i64, C.c_int, vp, vp]
    lib.nzhip_tensorcore_gemm.argtypes = [vp, vp, vp, shape, shape, shape, vp]
    lib.nzhip_im2col.argtypes = [vp, vp] + [sz] * 10 + [vp]
    lib.nzhip_col2im.argtypes = [vp, vp, sz, sz, sz, sz, vp]
    lib.nzhip_conv2d_forward.argtypes = [vp, vp, vp, vp] + [sz] * 10 + [i64, i64, C.c_int, vp]
    lib.nzhip_conv2d_backward_data.argtypes = [vp, vp, vp] + [sz] * 10 + [C.c_int, vp]
    lib.nzhip_conv2d_backward_weights.argtypes = [vp, vp, vp] + [sz] * 10 + [vp]
    lib.nzhip_add_broadcast.argtypes = [vp, vp, vp, shape, shape, shape, vp]
    lib.nzhip_relu.argtypes = [vp, vp, sz, vp]
    lib.nzhip_fill.argtypes = [vp, C.c_float, sz, vp]
    lib.nzhip_gemm_backward.argtypes = [vp, vp, vp, shape, shape, shape, vp]
    lib.nzhip_matmul_backward.argtypes = [vp, vp, vp, vp, vp, shape, shape, shape, vp]
    lib.nzhip_relu_backward.argtypes = [vp, vp, vp, sz, vp]
    lib.nzhip_add_backward.argtypes = [vp, vp, shape, shape, vp]
    lib.nzhip_im2col_backward.argtypes = [vp, vp] + [sz] * 10 + [vp]
    lib.nzhip_col2im_backward.argtypes = [vp, vp, sz, sz, sz, sz, vp]
    lib.nzhip_matmul_f32.argtypes = [vp, vp, vp, shape, shape, shape, vp]
    lib.nzhip_sgd_step.argtypes = [vp, vp, C.c_float, sz, vp]
    lib.nzhip_softmax.argtypes = [vp, vp, sz, sz, vp]
    lib.nzhip_softmax_jacobian.argtypes = [vp, vp, sz, sz, vp]
    lib.nzhip_softmax_backward.argtypes = [vp, vp, vp, sz, sz, vp]
    lib.nzhip_conv2d_backward_bias.argtypes = [vp, vp, sz, sz, sz, vp]
    lib.nzhip_conv2d_backward_relu_bias.argtypes = [vp, vp, vp, vp, sz, sz, sz, vp]
    lib.nzhip_avgpool2d.argtypes = [vp, vp] + [sz] * 9 + [vp]
    lib.nzhip_avgpool2d_backward.argtypes = [vp, vp] + [sz] * 9 + [vp]
    lib.nzhip_avgpool2d_backward_overwrite.argtypes = [vp, vp] + [sz] * 9 + [vp]
    lib.nzhip_bce_loss.argtypes = [vp, vp, vp, sz, vp]
    lib.nzhip_bce_backward.argtypes = [vp, vp, vp, sz, vp]
    lib.nzhip_mse_loss.argtypes = [vp, vp, vp, sz, vp]
    lib.nzhip_mse_backward.argtypes = [vp, vp, vp, sz, vp]
    lib.nzhip_expand.argtypes = [vp, vp, sz, sz, vp]
    lib.nzhip_compress.argtypes = [vp, vp, sz, sz, vp]
    lib.nzhip_adam_step.argtypes = [vp, vp, vp, vp, C.c_float, C.c_float, C.c_float, C.c_float, C.c_int, sz, vp]
    lib.nzhip_fill_many.argtypes = [C.c_int, vp, vp, C.c_float, vp]
    lib.nzhip_sgd_step_many.argtypes = [C.c_int, vp, vp, vp, C.c_float, vp]
    lib.nzhip_adam_step_many.argtypes = [C.c_int, vp, vp, vp, vp, vp, vp, C.c_float, C.c_float, C.c_float, C.c_float, vp]
    lib.nzhip_default_stream.restype = vp
    lib.nzhip_malloc.argtypes = [C.POINTER(vp), sz]
    lib.nzhip_free_async.argtypes = [vp]
    lib.nzhip_free.argtypes = [vp]
    lib.nzhip_host_malloc.argtypes = [C.POINTER(vp), sz]
    lib.nzhip_host_free.argtypes = [vp]
    lib.nzhip_memset.argtypes = [vp, C.c_int, sz]
    for n in ("nzhip_memcpy_h2d", "nzhip_memcpy_d2d", "nzhip_memcpy_d2h"):
        getattr(lib, n).argtypes = [vp, vp, sz]
    lib.nzhip_sync_ptr.argtypes = [vp]
    lib.nzhip_stream_wait.argtypes = [vp]
    lib.nzhip_allocator_stats.argtypes = [C.POINTER(sz), C.POINTER(sz), C.POINTER(sz)]
    _LIB = lib
    return lib


def check(status: int) -> None:
    if status != 0:
        raise NzHipError(status, load().nzhip_last_error().decode(errors="replace"))


def shape4(s) -> C.Array:
    return (C.c_size_t * 4)(*[int(v) for v in s])


# --------------------------------------------------------------------------------------------
# Torch-facing helpers. torch is used for device memory and streams only.
# --------------------------------------------------------------------------------------------
def _stream_handle(stream=None) -> int:
    import torch
    s = stream if stream is not None else torch.cuda.current_stream()
    return int(s.cuda_stream)


def _dev(t):
    import torch
    # page-locked host tensors are mapped into the device at the same address and are legal operands
    assert (t.is_cuda or t.is_pinned()) and t.dtype == torch.float32 and t.is_contiguous(), \
        "expects contiguous fp32 CUDA (or pinned host) tensors"
    return t.data_ptr()


class Prepared:
    """A prepared-operand handle (nzhip_prepared): owns the fp16 image of a weight operand between calls."""

    def __init__(self):
        self._h = C.c_void_p()
        check(load().nzhip_prepared_create(C.byref(self._h)))

    @property
    def handle(self):
        return self._h

    def invalidate(self):
        check(load().nzhip_prepared_invalidate(self._h))

    def fills(self) -> int:
        n = C.c_ulonglong(0)
        check(load().nzhip_prepared_fills(self._h, C.byref(n)))
        return n.value

    def close(self):
        if self._h:
            check(load().nzhip_prepared_destroy(self._h))
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def gemm(A, B, *, a_trans=False, b_trans=False, bias=None, bias_strides=(0, 0), relu=False, out=None,
         force_tile=0, stream=None, static=False, prepared_b=None):
    """C = act(f16(A) @ f16(B) + bias) for 2-D tensors. a_trans: A holds K x M; b_trans: B holds N x K.
    bias_strides = (row stride, column stride) in elements. static: through nzhip_gemm_static (the
    entry point that allocates nothing); `out` must then be given."""
    import torch
    lib = load()
    M, K = (A.shape[1], A.shape[0]) if a_trans else A.shape
    N = B.shape[0] if b_trans else B.shape[1]
    assert (B.shape[1] if b_trans else B.shape[0]) == K
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=A.device)
    d = GemmDesc()
    d.A, d.B, d.C = _dev(A), _dev(B), _dev(out)
    d.M, d.N, d.K = M, N, K
    d.lda, d.ldb, d.ldc = A.shape[1], B.shape[1], N
    d.a_layout = LAYOUT_TRANS if a_trans else LAYOUT_ROW
    d.b_layout = LAYOUT_TRANS if b_trans else LAYOUT_ROW
    d.batch_n = d.batch_c = 1
    if bias is not None:
        d.bias = _dev(bias)
        d.bias_stride_row, d.bias_stride_col = bias_strides
    d.activation = ACT_RELU if relu else ACT_NONE
    if prepared_b is not None:
        check(lib.nzhip_gemm_prepared_b(C.byref(d), prepared_b.handle, _stream_handle(stream)))
    elif static:
        check(lib.nzhip_gemm_static(C.byref(d), _stream_handle(stream)))
    elif force_tile:
        check(lib.nzhip_gemm_force_tile(C.byref(d), force_tile, _stream_handle(stream)))
    else:
        check(lib.nzhip_gemm(C.byref(d), _stream_handle(stream)))
    return out


def prepare_gemm(A, B, out, *, a_trans=False, b_trans=False, bias=None, bias_strides=(0, 0), relu=False, stream=None,
                 prepared_b=None):
    """Build the descriptor once and return a zero-argument callable that only enqueues the
    product (for timing loops, where per-call Python work would otherwise dominate small shapes)."""
    lib = load()
    M, K = (A.shape[1], A.shape[0]) if a_trans else A.shape
    N = B.shape[0] if b_trans else B.shape[1]
    d = GemmDesc()
    d.A, d.B, d.C = _dev(A), _dev(B), _dev(out)
    d.M, d.N, d.K = M, N, K
    d.lda, d.ldb, d.ldc = A.shape[1], B.shape[1], N
    d.a_layout = LAYOUT_TRANS if a_trans else LAYOUT_ROW
    d.b_layout = LAYOUT_TRANS if b_trans else LAYOUT_ROW
    d.batch_n = d.batch_c = 1
    if bias is not None:
        d.bias = _dev(bias)
        d.bias_stride_row, d.bias_stride_col = bias_strides
    d.activation = ACT_RELU if relu else ACT_NONE
    ref, h, fn = C.byref(d), C.c_void_p(_stream_handle(stream)), lib.nzhip_gemm
    if prepared_b is not None:
        pb, fp = prepared_b.handle, lib.nzhip_gemm_prepared_b

        def call_prepared(_keep=(d, A, B, out, bias, prepared_b)):
            st = fp(ref, pb, h)
            if st:
                check(st)
        return call_prepared

    def call(_keep=(d, A, B, out, bias)):
        st = fn(ref, h)
        if st:
            check(st)
    return call


def tensorcore_gemm(A, B, out=None, stream=None):
    """4-D batched/broadcast product with the semantics of nz::data::iTensorCoreGEMM."""
    import torch
    lib = load()
    sa, sb = tuple(A.shape), tuple(B.shape)
    sc = (max(sa[0], sb[0]), max(sa[1], sb[1]), sa[2], sb[3])
    if out is None:
        out = torch.empty(sc, dtype=torch.float32, device=A.device)
    check(lib.nzhip_tensorcore_gemm(_dev(A), _dev(B), _dev(out), shape4(sa), shape4(sb), shape4(tuple(out.shape)),
                                    _stream_handle(stream)))
    return out


def im2col(x, K_h, K_w, stride, pad, stream=None):
    import torch
    lib = load()
    N, Cc, H, W = x.shape
    Ho, Wo = (H + 2 * pad - K_h) // stride + 1, (W + 2 * pad - K_w) // stride + 1
    out = torch.empty((N, 1, Ho * Wo, Cc * K_h * K_w), dtype=torch.float32, device=x.device)
    check(lib.nzhip_im2col(_dev(out), _dev(x), Ho, Wo, Cc, K_h, K_w, stride, pad, H, W, N, _stream_handle(stream)))
    return out


def col2im(col, Ho, Wo, stream=None):
    import torch
    lib = load()
    N, _, HW, O = col.shape
    out = torch.empty((N, O, Ho, Wo), dtype=torch.float32, device=col.device)
    check(lib.nzhip_col2im(_dev(out), _dev(col), Ho, Wo, O, N, _stream_handle(stream)))
    return out


def conv2d_forward(x, w_ref, bias, K_h, K_w, stride, pad, *, bias_strides=(0, 1), relu=False, out=None, stream=None,
                   prepared_w=None):
    """x [N,C,H,W]; w_ref [Wb,1,C*Kh*Kw,O]; bias_strides = (pixel stride, channel stride)."""
    import torch
    lib = load()
    N, Cc, H, W = x.shape
    Wb, _, CKK, O = w_ref.shape
    assert CKK == Cc * K_h * K_w
    Ho, Wo = (H + 2 * pad - K_h) // stride + 1, (W + 2 * pad - K_w) // stride + 1
    if out is None:
        out = torch.empty((N, O, Ho, Wo), dtype=torch.float32, device=x.device)
    if prepared_w is not None:
        check(lib.nzhip_conv2d_forward_prepared(_dev(out), _dev(x), _dev(w_ref), None if bias is None else _dev(bias), N, Cc,
                                                H, W, O, K_h, K_w, stride, pad, Wb, bias_strides[0], bias_strides[1],
                                                ACT_RELU if relu else ACT_NONE, prepared_w.handle, _stream_handle(stream)))
        return out
    check(lib.nzhip_conv2d_forward(_dev(out), _dev(x), _dev(w_ref), None if bias is None else _dev(bias), N, Cc, H, W,
                                   O, K_h, K_w, stride, pad, Wb, bias_strides[0], bias_strides[1],
                                   ACT_RELU if relu else ACT_NONE, _stream_handle(stream)))
    return out


def add_broadcast(a, b, stream=None):
    import torch
    lib = load()
    so = (max(a.shape[0], b.shape[0]), max(a.shape[1], b.shape[1]), a.shape[2], a.shape[3])
    out = torch.empty(so, dtype=torch.float32, device=a.device)
    check(lib.nzhip_add_broadcast(_dev(out), _dev(a), _dev(b), shape4(so), shape4(a.shape), shape4(b.shape),
                                  _stream_handle(stream)))
    return out


def fill(a, value, stream=None):
    lib = load()
    check(lib.nzhip_fill(_dev(a), float(value), a.numel(), _stream_handle(stream)))
    return a


def relu(a, stream=None):
    import torch
    lib = load()
    out = torch.empty_like(a)
    check(lib.nzhip_relu(_dev(out), _dev(a), a.numel(), _stream_handle(stream)))
    return out


# ---- backward of the path (gradient buffers are updated in place, as in the reference) ----------
def gemm_backward(A, B, C, stream=None):
    """C[n or 0][c or 0] += f16(A)·f16(B) over the batch max(A, B); C is modified in place."""
    lib = load()
    check(lib.nzhip_gemm_backward(_dev(A), _dev(B), _dev(C), shape4(A.shape), shape4(B.shape), shape4(C.shape),
                                  _stream_handle(stream)))
    return C


def matmul_backward(dA, dB, A, B, dC, stream=None):
    """dA += dC·Bᵀ, dB += Aᵀ·dC in place; pass None for a gradient that is not wanted."""
    lib = load()
    check(lib.nzhip_matmul_backward(None if dA is None else _dev(dA), None if dB is None else _dev(dB), _dev(A), _dev(B),
                                    _dev(dC), shape4(A.shape), shape4(B.shape), shape4(dC.shape), _stream_handle(stream)))
    return dA, dB


def relu_backward(x, dy, stream=None):
    import torch
    lib = load()
    dx = torch.empty_like(x)
    check(lib.nzhip_relu_backward(_dev(dx), _dev(x), _dev(dy), x.numel(), _stream_handle(stream)))
    return dx


def add_backward(din, dout, stream=None):
    lib = load()
    check(lib.nzhip_add_backward(_dev(din), _dev(dout), shape4(din.shape), shape4(dout.shape), _stream_handle(stream)))
    return din


def im2col_backward(dx, dcol, K_h, K_w, stride, pad, stream=None):
    lib = load()
    N, Cc, H, W = dx.shape
    Ho, Wo = (H + 2 * pad - K_h) // stride + 1, (W + 2 * pad - K_w) // stride + 1
    check(lib.nzhip_im2col_backward(_dev(dx), _dev(dcol), Ho, Wo, Cc, K_h, K_w, stride, pad, H, W, N, _stream_handle(stream)))
    return dx


def conv2d_backward_data(dx, dy, w_ref, K_h, K_w, stride, pad, *, accumulate=True, stream=None):
    """dx (+)= gradient of conv2d_forward with respect to x; dx [N,C,H,W], dy [N,O,H_out,W_out]."""
    lib = load()
    N, Cc, H, W = dx.shape
    check(lib.nzhip_conv2d_backward_data(_dev(dx), _dev(dy), _dev(w_ref), N, Cc, H, W, dy.shape[1], K_h, K_w, stride, pad,
                                         w_ref.shape[0], 1 if accumulate else 0, _stream_handle(stream)))
    return dx


def conv2d_backward_weights(dw, x, dy, K_h, K_w, stride, pad, stream=None):
    """dw += gradient of conv2d_forward with respect to w_ref; dw [w_batch,1,C*K_h*K_w,O] is modified in place."""
    lib = load()
    N, Cc, H, W = x.shape
    check(lib.nzhip_conv2d_backward_weights(_dev(dw), _dev(x), _dev(dy), N, Cc, H, W, dy.shape[1], K_h, K_w, stride, pad,
                                            dw.shape[0], _stream_handle(stream)))
    return dw


def col2im_backward(dy, stream=None):
    import torch
    lib = load()
    N, O, Ho, Wo = dy.shape
    out = torch.empty((N, 1, Ho * Wo, O), dtype=torch.float32, device=dy.device)
    check(lib.nzhip_col2im_backward(_dev(out), _dev(dy), Ho, Wo, O, N, _stream_handle(stream)))
    return out


# ---- fp32-exact matmul and optimizer steps ---------------------------------------------------------
def matmul_f32(A, B, out=None, stream=None):
    import torch
    lib = load()
    so = (max(A.shape[0], B.shape[0]), max(A.shape[1], B.shape[1]), A.shape[2], B.shape[3])
    if out is None:
        out = torch.empty(so, dtype=torch.float32, device=A.device)
    check(lib.nzhip_matmul_f32(_dev(A), _dev(B), _dev(out), shape4(A.shape), shape4(B.shape), shape4(so), _stream_handle(stream)))
    return out


def sgd_step(data, grad, lr, stream=None):
    lib = load()
    check(lib.nzhip_sgd_step(_dev(data), _dev(grad), lr, data.numel(), _stream_handle(stream)))
    return data


def adam_step(data, m, v, grad, lr, beta1, beta2, eps, t, stream=None):
    lib = load()
    check(lib.nzhip_adam_step(_dev(data), _dev(m), _dev(v), _dev(grad), lr, beta1, beta2, eps, t, data.numel(),
                              _stream_handle(stream)))
    return data, m, v


def _pointer_array(tensors):
    return (C.c_void_p * len(tensors))(*[_dev(t) for t in tensors])


def _count_array(tensors):
    return (C.c_size_t * len(tensors))(*[t.numel() for t in tensors])


def fill_many(tensors, value, stream=None):
    """nzhip_fill for a list of tensors in one launch per NZHIP_MANY_MAX of them."""
    lib = load()
    check(lib.nzhip_fill_many(len(tensors), _pointer_array(tensors), _count_array(tensors), float(value), _stream_handle(stream)))
    return tensors


def sgd_step_many(datas, grads, lr, stream=None):
    lib = load()
    check(lib.nzhip_sgd_step_many(len(datas), _pointer_array(datas), _pointer_array(grads), _count_array(datas), lr,
                                  _stream_handle(stream)))
    return datas


def adam_step_many(datas, ms, vs, grads, ts, lr, beta1, beta2, eps, stream=None):
    """ts[k]: the step count of tensor k (>= 1)."""
    lib = load()
    check(lib.nzhip_adam_step_many(len(datas), _pointer_array(datas), _pointer_array(ms), _pointer_array(vs), _pointer_array(grads),
                                   _count_array(datas), (C.c_int * len(ts))(*ts), lr, beta1, beta2, eps, _stream_handle(stream)))
    return datas, ms, vs


def softmax(x, stream=None):
    import torch
    lib = load()
    out = torch.empty_like(x)
    check(lib.nzhip_softmax(_dev(out), _dev(x), x.shape[2] * x.shape[3], x.shape[0] * x.shape[1], _stream_handle(stream)))
    return out


def softmax_jacobian(s, stream=None):
    import torch
    lib = load()
    n = max(s.shape[2], s.shape[3])
    out = torch.empty((s.shape[0], s.shape[1], n, n), dtype=torch.float32, device=s.device)
    check(lib.nzhip_softmax_jacobian(_dev(out), _dev(s), n, s.shape[0] * s.shape[1], _stream_handle(stream)))
    return out


def softmax_backward(s, dy, stream=None):
    """SoftmaxNode::backward in one kernel (no Jacobian in memory)."""
    import torch
    lib = load()
    dx = torch.empty_like(s)
    check(lib.nzhip_softmax_backward(_dev(dx), _dev(s), _dev(dy), s.shape[2] * s.shape[3], s.shape[0] * s.shape[1],
                                     _stream_handle(stream)))
    return dx


def softmax_backward_gemm(s, dy, stream=None):
    """SoftmaxNode::backward as the reference spells it: Jacobian times gradient through the fp16 GEMM entry."""
    jac = softmax_jacobian(s, stream)
    return tensorcore_gemm(jac, dy, stream=stream) if s.shape[2] > s.shape[3] else tensorcore_gemm(dy, jac, stream=stream)


def conv2d_backward_bias(dbias, dz, stream=None):
    """dbias [1,1,HW,O] += sum over n of dz [N,O,H,W] (transposed); modified in place."""
    lib = load()
    N, O, H, W = dz.shape
    check(lib.nzhip_conv2d_backward_bias(_dev(dbias), _dev(dz), N, O, H * W, _stream_handle(stream)))
    return dbias


def conv2d_backward_relu_bias(dbias, y, dy, stream=None):
    """Returns dz = dy where y > 0 else 0, and adds its transposed batch sum onto dbias [1,1,HW,O] in place."""
    import torch
    lib = load()
    N, O, H, W = dy.shape
    dz = torch.empty_like(dy)
    check(lib.nzhip_conv2d_backward_relu_bias(_dev(dz), _dev(dbias), _dev(y), _dev(dy), N, O, H * W, _stream_handle(stream)))
    return dz


def avgpool2d(x, pool, stride, pad, stream=None):
    import torch
    lib = load()
    N, Cc, H, W = x.shape
    ok = stride > 0 and H + 2 * pad >= pool and W + 2 * pad >= pool       # otherwise the library rejects the call
    Ho, Wo = ((H + 2 * pad - pool) // stride + 1, (W + 2 * pad - pool) // stride + 1) if ok else (1, 1)
    out = torch.empty((N, Cc, Ho, Wo), dtype=torch.float32, device=x.device)
    check(lib.nzhip_avgpool2d(_dev(out), _dev(x), pool, stride, pad, N, Cc, H, W, Ho, Wo, _stream_handle(stream)))
    return out


def avgpool2d_backward(dx, dy, pool, stride, pad, stream=None, overwrite=False):
    """dx += gradient of avgpool2d (overwrite: dx = it, dx's old contents are not read); dx has the input's shape, dy the output's."""
    lib = load()
    N, Cc, H, W = dx.shape
    fn = lib.nzhip_avgpool2d_backward_overwrite if overwrite else lib.nzhip_avgpool2d_backward
    check(fn(_dev(dx), _dev(dy), pool, stride, pad, N, Cc, H, W, dy.shape[2], dy.shape[3], _stream_handle(stream)))
    return dx


def bce_loss(predict, real, stream=None):
    """Device scalar (a 1-element tensor) holding the mean binary cross-entropy."""
    import torch
    lib = load()
    loss = torch.empty(1, dtype=torch.float32, device=predict.device)
    check(lib.nzhip_bce_loss(_dev(loss), _dev(predict), _dev(real), predict.numel(), _stream_handle(stream)))
    return loss


def bce_backward(predict, real, stream=None):
    import torch
    lib = load()
    grad = torch.empty_like(predict)
    check(lib.nzhip_bce_backward(_dev(grad), _dev(predict), _dev(real), predict.numel(), _stream_handle(stream)))
    return grad


def mse_loss(predict, real, stream=None):
    import torch
    lib = load()
    loss = torch.empty(1, dtype=torch.float32, device=predict.device)
    check(lib.nzhip_mse_loss(_dev(loss), _dev(predict), _dev(real), predict.numel(), _stream_handle(stream)))
    return loss


def mse_backward(predict, real, stream=None):
    import torch
    lib = load()
    grad = torch.empty_like(predict)
    check(lib.nzhip_mse_backward(_dev(grad), _dev(predict), _dev(real), predict.numel(), _stream_handle(stream)))
    return grad


def expand(x, batches, stream=None):
    import torch
    lib = load()
    out = torch.empty((batches,) + tuple(x.shape[1:]), dtype=torch.float32, device=x.device)
    check(lib.nzhip_expand(_dev(out), _dev(x), x.numel(), batches, _stream_handle(stream)))
    return out


def compress(out, x, stream=None):
    """out[0] += sum over the batch of x."""
    lib = load()
    check(lib.nzhip_compress(_dev(out), _dev(x), out.numel(), x.shape[0], _stream_handle(stream)))
    return out
