"""ctypes loader and numpy wrappers for the CPU oracle (libnz_oracle_*.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke()`` and
by the ``cpu_baseline`` leg of ``bench.py`` -- never by the shipped library.
Each wrapper mirrors one function of ``nz_oracle.h``; the reference file:line
each one restates is cited there.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_AVX512 = ("avx512f", "avx512bw", "avx512cd", "avx512dq", "avx512vl")


def _cpu_flags() -> set:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("flags"):
                    return set(line.split(":", 1)[1].split())
    except OSError:
        pass
    return set()


def build(force: bool = False) -> None:
    """Compile both ISA variants with the committed Makefile."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE, "-j2"], stdout=subprocess.DEVNULL)


def _load() -> C.CDLL:
    flags = _cpu_flags()
    order = ["libnz_oracle_v4.so", "libnz_oracle_v3.so"] if all(f in flags for f in _AVX512) else ["libnz_oracle_v3.so"]
    if os.environ.get("NZ_ORACLE_ISA") == "v3":
        order = ["libnz_oracle_v3.so"]
    sources = [os.path.join(_HERE, f) for f in ("nz_oracle.c", "nz_oracle.h", "Makefile")]
    newest = max(os.path.getmtime(f) for f in sources if os.path.exists(f))
    for name in order:
        path = os.path.join(_HERE, name)
        if os.path.exists(path) and os.path.getmtime(path) >= newest:       # built, and not older than its sources
            return C.CDLL(path)
    build()
    return C.CDLL(os.path.join(_HERE, order[-1]))


_lib = _load()

_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_f64p = np.ctypeslib.ndpointer(dtype=np.float64, flags="C_CONTIGUOUS")
_sz = C.c_size_t
_Shape = _sz * 4


def _sig(name, restype, *argtypes):
    fn = getattr(_lib, name)
    fn.restype = restype
    fn.argtypes = list(argtypes)
    return fn


_f32_to_f16_bits = _sig("nzo_f32_to_f16_bits", C.c_uint16, C.c_float)
_f16_bits_to_f32 = _sig("nzo_f16_bits_to_f32", C.c_float, C.c_uint16)
_round_arr = _sig("nzo_round_f16_array", None, _f32p, _f32p, _sz)
_gemm32 = _sig("nzo_gemm_f16in_f32acc", None, _f32p, _f32p, _f32p, _sz, _sz, _sz, _sz, _sz, _sz, C.c_int)
_gemm64 = _sig("nzo_gemm_f16in_f64acc", None, _f32p, _f32p, _f64p, _sz, _sz, _sz, _sz, _sz, _sz, C.c_int)
_gemm_rows = _sig("nzo_gemm_rows", None, _f32p, _f32p, C.c_void_p, C.c_void_p, _sz, _sz, _sz, _sz, _sz, _sz, C.c_int)
_tc_gemm = _sig("nzo_tensorcore_gemm", None, _f32p, _f32p, _f32p, _Shape, _Shape, _Shape)
_gen_mm = _sig("nzo_general_matmul", None, _f32p, _f32p, _f32p, _Shape, _Shape, _Shape)
_im2col = _sig("nzo_im2col", None, _f32p, _f32p, *([_sz] * 10))
_col2im = _sig("nzo_col2im", None, _f32p, _f32p, _sz, _sz, _sz, _sz)
_madd = _sig("nzo_matrix_add", None, _f32p, _f32p, _f32p, _Shape, _Shape, _Shape)
_relu = _sig("nzo_relu", None, _f32p, _f32p, _sz)
_gemm_bwd = _sig("nzo_gemm_backward", None, _f32p, _f32p, _f32p, _Shape, _Shape, _Shape)
_matmul_bwd = _sig("nzo_matmul_backward", None, C.c_void_p, C.c_void_p, _f32p, _f32p, _f32p, _Shape, _Shape, _Shape)
_relu_bwd = _sig("nzo_relu_backward", None, _f32p, _f32p, _f32p, _sz)
_add_bwd = _sig("nzo_add_backward", None, _f32p, _f32p, _Shape, _Shape)
_im2col_bwd = _sig("nzo_im2col_backward", None, _f32p, _f32p, *([_sz] * 10))
_col2im_bwd = _sig("nzo_col2im_backward", None, _f32p, _f32p, _sz, _sz, _sz, _sz)
_conv_bwd_data = _sig("nzo_conv2d_backward_data_strided", None, _f32p, _f32p, _f32p, *([_sz] * 10))
_conv_bwd_w = _sig("nzo_conv2d_backward_weights_strided", None, _f32p, _f32p, _f32p, *([_sz] * 10))
_softmax = _sig("nzo_softmax", None, _f32p, _f32p, _sz, _sz)
_softmax_jac = _sig("nzo_softmax_jacobian", None, _f32p, _f32p, _sz, _sz)
_avgpool = _sig("nzo_avgpool2d", None, _f32p, _f32p, *([_sz] * 9))
_avgpool_bwd = _sig("nzo_avgpool2d_backward", None, _f32p, _f32p, *([_sz] * 9))
_bce = _sig("nzo_bce_loss", C.c_float, _f32p, _f32p, _sz)
_bce_bwd = _sig("nzo_bce_backward", None, _f32p, _f32p, _f32p, _sz)
_mse = _sig("nzo_mse_loss", C.c_float, _f32p, _f32p, _sz)
_mse_bwd = _sig("nzo_mse_backward", None, _f32p, _f32p, _f32p, _sz)
_expand = _sig("nzo_expand", None, _f32p, _f32p, _sz, _sz)
_compress = _sig("nzo_compress", None, _f32p, _f32p, _sz, _sz)
_sgd = _sig("nzo_sgd_step", None, _f32p, _f32p, C.c_float, _sz)
_adam = _sig("nzo_adam_step", None, _f32p, _f32p, _f32p, _f32p, C.c_float, C.c_float, C.c_float, C.c_float, C.c_int, _sz)
_conv_graph = _sig("nzo_conv2d_graph", None, _f32p, _f32p, _f32p, C.c_void_p, *([_sz] * 10), C.c_int)
_conv_direct = _sig("nzo_conv2d_direct_f64", None, _f64p, _f32p, _f32p, C.c_void_p, *([_sz] * 9), C.c_int)
_linear = _sig("nzo_linear_graph", None, _f32p, _f32p, _f32p, C.c_void_p, _sz, _sz, _sz, C.c_int)
_errors = _sig("nzo_errors_f32_vs_f64", None, _f32p, _f64p, _sz, C.c_double, C.POINTER(C.c_double), C.POINTER(C.c_double))
_fill = _sig("nzo_fill", None, _f32p, _sz, C.c_uint64, C.c_int, C.c_double, C.c_double)
_nthreads = _sig("nzo_num_threads", C.c_int)
_set_nthreads = _sig("nzo_set_num_threads", None, C.c_int)
_f16c_hw = _sig("nzo_f16c_hw_bits", C.c_uint16, C.c_uint32)
_f16c_range = _sig("nzo_f16c_compare_range", C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64, C.POINTER(C.c_uint32))
_f16c_widen = _sig("nzo_f16c_compare_widen", C.c_uint32)


def _c(a, dtype=np.float32):
    return np.ascontiguousarray(a, dtype=dtype)


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


# ---- fp16 rounding ---------------------------------------------------------
def f32_to_f16_bits(x: float) -> int:
    return int(_f32_to_f16_bits(x))


def f16_bits_to_f32(h: int) -> float:
    return float(_f16_bits_to_f32(h))


def round_f16(a: np.ndarray) -> np.ndarray:
    a = _c(a)
    out = np.empty_like(a)
    _round_arr(out.reshape(-1), a.reshape(-1), a.size)
    return out


def f16c_hw_bits(fbits: int) -> int:
    return int(_f16c_hw(fbits))


def f16c_compare_range(start: int, count: int, step: int = 1):
    first = C.c_uint32(0)
    bad = _f16c_range(start, count, step, C.byref(first))
    return int(bad), int(first.value)


def f16c_compare_widen() -> int:
    return int(_f16c_widen())


# ---- GEMM ------------------------------------------------------------------
def gemm(A: np.ndarray, B: np.ndarray, trans_b: bool = False) -> np.ndarray:
    """C = f16(A) @ f16(B) with fp32 accumulation (k ascending). 2-D operands."""
    A, B = _c(A), _c(B)
    M, K = A.shape
    N = B.shape[0] if trans_b else B.shape[1]
    assert (B.shape[1] if trans_b else B.shape[0]) == K
    out = np.empty((M, N), np.float32)
    _gemm32(A, B, out, M, N, K, A.shape[1], B.shape[1], N, int(trans_b))
    return out


def gemm_f64(A: np.ndarray, B: np.ndarray, trans_b: bool = False) -> np.ndarray:
    A, B = _c(A), _c(B)
    M, K = A.shape
    N = B.shape[0] if trans_b else B.shape[1]
    out = np.empty((M, N), np.float64)
    _gemm64(A, B, out, M, N, K, A.shape[1], B.shape[1], N, int(trans_b))
    return out


def gemm_rows(A: np.ndarray, B: np.ndarray, row0: int, nrows: int, trans_b: bool = False, want32=True, want64=True):
    A, B = _c(A), _c(B)
    K = A.shape[1]
    N = B.shape[0] if trans_b else B.shape[1]
    c32 = np.empty((nrows, N), np.float32) if want32 else None
    c64 = np.empty((nrows, N), np.float64) if want64 else None
    _gemm_rows(A, B, _ptr(c32), _ptr(c64), row0, nrows, N, K, A.shape[1], B.shape[1], int(trans_b))
    return c32, c64


def tensorcore_gemm(A: np.ndarray, B: np.ndarray) -> np.ndarray:
    """Batched/broadcast 4-D GEMM exactly as TensorCoreGEMMParallel loops it."""
    A, B = _c(A), _c(B)
    sa, sb = A.shape, B.shape
    sc = (max(sa[0], sb[0]), max(sa[1], sb[1]), sa[2], sb[3])
    out = np.empty(sc, np.float32)
    _tc_gemm(A.reshape(-1), B.reshape(-1), out.reshape(-1), _Shape(*sa), _Shape(*sb), _Shape(*sc))
    return out


def general_matmul(A: np.ndarray, B: np.ndarray) -> np.ndarray:
    A, B = _c(A), _c(B)
    sa, sb = A.shape, B.shape
    sc = (max(sa[0], sb[0]), max(sa[1], sb[1]), sa[2], sb[3])
    out = np.empty(sc, np.float32)
    _gen_mm(A.reshape(-1), B.reshape(-1), out.reshape(-1), _Shape(*sa), _Shape(*sb), _Shape(*sc))
    return out


# ---- conv lowering pieces ---------------------------------------------------
def out_hw(H, W, K_h, K_w, stride, pad):
    return (H + 2 * pad - K_h) // stride + 1, (W + 2 * pad - K_w) // stride + 1


def im2col(x: np.ndarray, K_h: int, K_w: int, stride: int, pad: int) -> np.ndarray:
    x = _c(x)
    N, Cc, H, W = x.shape
    Ho, Wo = out_hw(H, W, K_h, K_w, stride, pad)
    out = np.empty((N, 1, Ho * Wo, Cc * K_h * K_w), np.float32)
    _im2col(out.reshape(-1), x.reshape(-1), Ho, Wo, Cc, K_h, K_w, stride, pad, H, W, N)
    return out


def col2im(col: np.ndarray, Ho: int, Wo: int) -> np.ndarray:
    col = _c(col)
    N, _, HW, O = col.shape
    assert HW == Ho * Wo
    out = np.empty((N, O, Ho, Wo), np.float32)
    _col2im(out.reshape(-1), col.reshape(-1), Ho, Wo, O, N)
    return out


def matrix_add(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    a, b = _c(a), _c(b)
    so = (max(a.shape[0], b.shape[0]), max(a.shape[1], b.shape[1]), a.shape[2], a.shape[3])
    out = np.empty(so, np.float32)
    _madd(out.reshape(-1), a.reshape(-1), b.reshape(-1), _Shape(*so), _Shape(*a.shape), _Shape(*b.shape))
    return out


def relu(a: np.ndarray) -> np.ndarray:
    a = _c(a)
    out = np.empty_like(a)
    _relu(out.reshape(-1), a.reshape(-1), a.size)
    return out


# ---- backward of the path ---------------------------------------------------
def gemm_backward(A: np.ndarray, B: np.ndarray, C_acc: np.ndarray) -> np.ndarray:
    """iGEMMBackward: returns C_acc + sum over the broadcast batch of f16(A)·f16(B) (C_acc is not modified)."""
    A, B = _c(A), _c(B)
    out = _c(C_acc).copy()
    _gemm_bwd(A.reshape(-1), B.reshape(-1), out.reshape(-1), _Shape(*A.shape), _Shape(*B.shape), _Shape(*out.shape))
    return out


def matmul_backward(A, B, dC, dA0=None, dB0=None):
    """MatMulNode::backward: (dA0 + dC·Bᵀ, dB0 + Aᵀ·dC); a gradient whose start value is None is skipped."""
    A, B, dC = _c(A), _c(B), _c(dC)
    dA = None if dA0 is None else _c(dA0).copy()
    dB = None if dB0 is None else _c(dB0).copy()
    _matmul_bwd(_ptr(dA), _ptr(dB), A.reshape(-1), B.reshape(-1), dC.reshape(-1), _Shape(*A.shape), _Shape(*B.shape),
                _Shape(*dC.shape))
    return dA, dB


def relu_backward(x: np.ndarray, dy: np.ndarray) -> np.ndarray:
    x, dy = _c(x), _c(dy)
    out = np.empty_like(x)
    _relu_bwd(out.reshape(-1), x.reshape(-1), dy.reshape(-1), x.size)
    return out


def add_backward(din0: np.ndarray, dout: np.ndarray) -> np.ndarray:
    """AddNode::backward for one input whose gradient currently holds din0."""
    out, dout = _c(din0).copy(), _c(dout)
    _add_bwd(out.reshape(-1), dout.reshape(-1), _Shape(*out.shape), _Shape(*dout.shape))
    return out


def im2col_backward(dx0: np.ndarray, dcol: np.ndarray, K_h: int, K_w: int, stride: int, pad: int) -> np.ndarray:
    out, dcol = _c(dx0).copy(), _c(dcol)
    N, Cc, H, W = out.shape
    Ho, Wo = out_hw(H, W, K_h, K_w, stride, pad)
    assert dcol.size == N * Ho * Wo * Cc * K_h * K_w
    _im2col_bwd(out.reshape(-1), dcol.reshape(-1), Ho, Wo, Cc, K_h, K_w, stride, pad, H, W, N)
    return out


def col2im_backward(dy: np.ndarray) -> np.ndarray:
    dy = _c(dy)
    N, O, Ho, Wo = dy.shape
    out = np.empty((N, 1, Ho * Wo, O), np.float32)
    _col2im_bwd(out.reshape(-1), dy.reshape(-1), Ho, Wo, O, N)
    return out


def conv2d_backward_weights(dw: np.ndarray, x: np.ndarray, dy: np.ndarray, K_h: int, K_w: int, pad: int, stride: int = 1) -> np.ndarray:
    """dw += gradient of the Conv2d graph with respect to its weights (in place, returns dw)."""
    x, dy = _c(x), _c(dy)
    assert dw.dtype == np.float32 and dw.flags.c_contiguous
    N, Cc, H, W = x.shape
    O = dy.shape[1]
    assert dy.shape == (N, O, (H + 2 * pad - K_h) // stride + 1, (W + 2 * pad - K_w) // stride + 1)
    assert dw.shape[1:] == (1, Cc * K_h * K_w, O)
    _conv_bwd_w(dw.reshape(-1), x.reshape(-1), dy.reshape(-1), N, Cc, H, W, O, K_h, K_w, stride, pad, dw.shape[0])
    return dw


def conv2d_backward_data(dx: np.ndarray, dy: np.ndarray, w_ref: np.ndarray, K_h: int, K_w: int, pad: int, stride: int = 1) -> np.ndarray:
    """dx += gradient of the Conv2d graph with respect to its input (in place, returns dx)."""
    dy, w_ref = _c(dy), _c(w_ref)
    assert dx.dtype == np.float32 and dx.flags.c_contiguous
    N, Cc, H, W = dx.shape
    O = dy.shape[1]
    assert dy.shape == (N, O, (H + 2 * pad - K_h) // stride + 1, (W + 2 * pad - K_w) // stride + 1) and w_ref.shape[2:] == (Cc * K_h * K_w, O)
    _conv_bwd_data(dx.reshape(-1), dy.reshape(-1), w_ref.reshape(-1), N, Cc, H, W, O, K_h, K_w, stride, pad, w_ref.shape[0])
    return dx


def softmax(x: np.ndarray) -> np.ndarray:
    """Softmax over the (h, w) vector of every (n, c); min(h, w) must be 1."""
    x = _c(x)
    out = np.empty_like(x)
    _softmax(out.reshape(-1), x.reshape(-1), x.shape[2] * x.shape[3], x.shape[0] * x.shape[1])
    return out


def softmax_jacobian(s: np.ndarray) -> np.ndarray:
    s = _c(s)
    n = max(s.shape[2], s.shape[3])
    out = np.empty((s.shape[0], s.shape[1], n, n), np.float32)
    _softmax_jac(out.reshape(-1), s.reshape(-1), n, s.shape[0] * s.shape[1])
    return out


def softmax_backward(s: np.ndarray, dy: np.ndarray) -> np.ndarray:
    """SoftmaxNode::backward (src/Nodes.cu:538-548): Jacobian times gradient through the fp16 GEMM."""
    jac = softmax_jacobian(s)
    return tensorcore_gemm(jac, dy) if s.shape[2] > s.shape[3] else tensorcore_gemm(dy, jac)


def avgpool2d(x: np.ndarray, pool: int, stride: int, pad: int) -> np.ndarray:
    x = _c(x)
    N, Cc, H, W = x.shape
    Ho, Wo = (H + 2 * pad - pool) // stride + 1, (W + 2 * pad - pool) // stride + 1
    out = np.empty((N, Cc, Ho, Wo), np.float32)
    _avgpool(out.reshape(-1), x.reshape(-1), pool, stride, pad, N, Cc, H, W, Ho, Wo)
    return out


def avgpool2d_backward(dx: np.ndarray, dy: np.ndarray, pool: int, stride: int, pad: int) -> np.ndarray:
    """Returns dx + gradient (dx has the input's shape)."""
    dx, dy = _c(dx).copy(), _c(dy)
    N, Cc, H, W = dx.shape
    _avgpool_bwd(dx.reshape(-1), dy.reshape(-1), pool, stride, pad, N, Cc, H, W, dy.shape[2], dy.shape[3])
    return dx


def bce_loss(predict: np.ndarray, real: np.ndarray) -> float:
    p, t = _c(predict), _c(real)
    return float(_bce(p.reshape(-1), t.reshape(-1), p.size))


def bce_backward(predict: np.ndarray, real: np.ndarray) -> np.ndarray:
    p, t = _c(predict), _c(real)
    g = np.empty_like(p)
    _bce_bwd(g.reshape(-1), p.reshape(-1), t.reshape(-1), p.size)
    return g


def mse_loss(predict: np.ndarray, real: np.ndarray) -> float:
    p, t = _c(predict), _c(real)
    return float(_mse(p.reshape(-1), t.reshape(-1), p.size))


def mse_backward(predict: np.ndarray, real: np.ndarray) -> np.ndarray:
    p, t = _c(predict), _c(real)
    g = np.empty_like(p)
    _mse_bwd(g.reshape(-1), p.reshape(-1), t.reshape(-1), p.size)
    return g


def expand(x: np.ndarray, batches: int) -> np.ndarray:
    x = _c(x)
    out = np.empty((batches,) + x.shape[1:], np.float32)
    _expand(out.reshape(-1), x.reshape(-1), x.size, batches)
    return out


def compress(out: np.ndarray, x: np.ndarray) -> np.ndarray:
    out, x = _c(out).copy(), _c(x)
    _compress(out.reshape(-1), x.reshape(-1), out.size, x.shape[0])
    return out


def sgd_step(data, grad, lr):
    out = _c(data).copy()
    _sgd(out.reshape(-1), _c(grad).reshape(-1), lr, out.size)
    return out


def adam_step(data, m, v, grad, lr, beta1, beta2, eps, t):
    """One Adam step; returns the new (data, m, v)."""
    d, m2, v2 = _c(data).copy(), _c(m).copy(), _c(v).copy()
    _adam(d.reshape(-1), m2.reshape(-1), v2.reshape(-1), _c(grad).reshape(-1), lr, beta1, beta2, eps, t, d.size)
    return d, m2, v2


def conv2d_graph(x, w_ref, bias_ref, K_h, K_w, stride, pad, relu=False) -> np.ndarray:
    """Model::Conv2d graph; w_ref is [Wb,1,C*Kh*Kw,O], bias_ref [1,1,Ho*Wo,O] or None."""
    x, w_ref = _c(x), _c(w_ref)
    N, Cc, H, W = x.shape
    Wb, _, CKK, O = w_ref.shape
    assert CKK == Cc * K_h * K_w and Wb in (1, N)
    Ho, Wo = out_hw(H, W, K_h, K_w, stride, pad)
    if bias_ref is not None:
        bias_ref = _c(bias_ref)
        assert bias_ref.size == Ho * Wo * O
    y = np.empty((N, O, Ho, Wo), np.float32)
    _conv_graph(y.reshape(-1), x.reshape(-1), w_ref.reshape(-1), _ptr(bias_ref), N, Cc, H, W, O, K_h, K_w, stride, pad,
                Wb, int(relu))
    return y


def conv2d_direct_f64(x, w_oihw, bias_o, stride, pad, relu=False) -> np.ndarray:
    x, w_oihw = _c(x), _c(w_oihw)
    N, Cc, H, W = x.shape
    O, C2, K_h, K_w = w_oihw.shape
    assert C2 == Cc
    if bias_o is not None:
        bias_o = _c(bias_o)
    Ho, Wo = out_hw(H, W, K_h, K_w, stride, pad)
    y = np.empty((N, O, Ho, Wo), np.float64)
    _conv_direct(y.reshape(-1), x.reshape(-1), w_oihw.reshape(-1), _ptr(bias_o), N, Cc, H, W, O, K_h, K_w, stride, pad,
                 int(relu))
    return y


def linear_graph(x, w_out_in, bias, relu=False) -> np.ndarray:
    x, w_out_in = _c(x), _c(w_out_in)
    batch, IN = x.shape
    OUT = w_out_in.shape[0]
    assert w_out_in.shape[1] == IN
    if bias is not None:
        bias = _c(bias)
    y = np.empty((batch, OUT), np.float32)
    _linear(y, x, w_out_in, _ptr(bias), batch, IN, OUT, int(relu))
    return y


# ---- helpers ----------------------------------------------------------------
def weights_oihw_to_ref(w_oihw: np.ndarray) -> np.ndarray:
    """OIHW -> the reference's [1,1,C*Kh*Kw,O] (row q = c*Kh*Kw + r*Kw + s; src/Model.cu:248-252)."""
    O = w_oihw.shape[0]
    return np.ascontiguousarray(w_oihw.reshape(O, -1).T, dtype=np.float32).reshape(1, 1, -1, O)


def bias_channel_to_ref(bias_o: np.ndarray, HW: int) -> np.ndarray:
    """Per-channel bias -> the reference's per-pixel-per-channel parameter [1,1,HW,O] (src/Model.cu:68-75)."""
    return np.ascontiguousarray(np.broadcast_to(bias_o.astype(np.float32)[None, :], (HW, bias_o.size))).reshape(1, 1, HW, -1)


def errors(got: np.ndarray, truth: np.ndarray, floor_abs: float):
    got = _c(got).reshape(-1)
    truth = _c(truth, np.float64).reshape(-1)
    mr, fr = C.c_double(0), C.c_double(0)
    _errors(got, truth, got.size, floor_abs, C.byref(mr), C.byref(fr))
    return mr.value, fr.value


def fill(shape, seed: int, kind: str = "uniform", lo: float = 0.0, hi: float = 1.0) -> np.ndarray:
    """kind 'uniform': U[lo,hi); 'normal': N(mean=lo, std=hi). Deterministic in (seed, n)."""
    out = np.empty(shape, np.float32)
    _fill(out.reshape(-1), out.size, seed, 0 if kind == "uniform" else 1, lo, hi)
    return out


def num_threads() -> int:
    return int(_nthreads())


def set_num_threads(n: int) -> None:
    _set_nthreads(n)
