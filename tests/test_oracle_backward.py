"""Pins the oracle's backward functions without running the reference: the reference's own literal
vectors (test/Test.cpp:820-903), its loop-nest specifications (:3011-3072, :3144-3177), and the
adjoint identity <J v, u> = <v, J^T u> that any correct backward of a linear map must satisfy."""
import numpy as np
import pytest


def test_matmul_backward_special_reference_vector(oracle):
    # test/Test.cpp:820-842: all-ones operands, n=2, c=3, m=2, k=3, p=2; A is [n,1,m,k], B is [1,c,k,p]
    n, c, m, k, p = 2, 3, 2, 3, 2
    A = np.ones((n, 1, m, k), np.float32)
    B = np.ones((1, c, k, p), np.float32)
    dC = np.ones((n, c, m, p), np.float32)
    dA, dB = oracle.matmul_backward(A, B, dC, np.zeros_like(A), np.zeros_like(B))
    assert np.array_equal(dA, np.full_like(A, 2 * c))
    assert np.array_equal(dB, np.full_like(B, 2 * n))


def test_matmul_backward_normal_reference_vector(oracle):
    # test/Test.cpp:844-903
    n, c, m, k, p = 2, 3, 2, 3, 2
    A = np.array([1, 2, 3, 4, 5, 6, 2, 3, 4, 5, 6, 7, 3, 4, 5, 6, 7, 8] * 2, np.float32).reshape(n, c, m, k)
    B = np.array([1, 4, 2, 5, 3, 6, 2, 5, 3, 6, 4, 7, 3, 6, 4, 7, 5, 8], np.float32).reshape(1, c, k, p)
    dC = np.ones((n, c, m, p), np.float32)
    Agrad = np.array([5, 7, 9, 5, 7, 9, 7, 9, 11, 7, 9, 11, 9, 11, 13, 9, 11, 13] * 2, np.float32).reshape(n, c, m, k)
    Bgrad = np.array([10, 10, 14, 14, 18, 18, 14, 14, 18, 18, 22, 22, 18, 18, 22, 22, 26, 26], np.float32).reshape(1, c, k, p)
    dA, dB = oracle.matmul_backward(A, B, dC, np.zeros_like(A), np.zeros_like(B))
    assert np.array_equal(dA, Agrad)
    assert np.array_equal(dB, Bgrad)


def test_gemm_backward_accumulates_onto_existing_gradient(oracle):
    rng = np.random.default_rng(3)
    A = rng.integers(-4, 5, (3, 1, 5, 7)).astype(np.float32)
    B = rng.integers(-4, 5, (1, 2, 7, 6)).astype(np.float32)
    C0 = rng.integers(-9, 10, (1, 1, 5, 6)).astype(np.float32)   # both batch dims reduce into one matrix
    want = C0.astype(np.float64).copy()
    for i in range(3):
        for j in range(2):
            want[0, 0] += A[i, 0].astype(np.float64) @ B[0, j].astype(np.float64)
    got = oracle.gemm_backward(A, B, C0)
    assert np.array_equal(got, want.astype(np.float32))           # integers: exact in any order


def test_matmul_backward_is_the_adjoint_of_forward(oracle):
    # <dC, A·B> differentiated: sum(dA*U) + sum(dB*V) == <dC, U·B + A·V> for integer data (exact)
    rng = np.random.default_rng(5)
    A = rng.integers(-3, 4, (2, 3, 4, 5)).astype(np.float32)
    B = rng.integers(-3, 4, (1, 3, 5, 6)).astype(np.float32)
    U = rng.integers(-3, 4, A.shape).astype(np.float32)
    V = rng.integers(-3, 4, B.shape).astype(np.float32)
    dC = rng.integers(-3, 4, (2, 3, 4, 6)).astype(np.float32)
    dA, dB = oracle.matmul_backward(A, B, dC, np.zeros_like(A), np.zeros_like(B))
    lhs = float((dA.astype(np.float64) * U).sum() + (dB.astype(np.float64) * V).sum())
    rhs = float((dC.astype(np.float64) * (oracle.tensorcore_gemm(U, B).astype(np.float64) + oracle.tensorcore_gemm(A, V))).sum())
    assert lhs == rhs


def test_matmul_backward_rounds_both_operands_to_fp16(oracle):
    # 1 + 2^-12 is not a half: a backward that skipped the rounding of dC or B would see it
    A = np.ones((1, 1, 1, 1), np.float32)
    B = np.full((1, 1, 1, 1), 1 + 2.0 ** -12, np.float32)
    dC = np.full((1, 1, 1, 1), 1 + 2.0 ** -12, np.float32)
    dA, dB = oracle.matmul_backward(A, B, dC, np.zeros_like(A), np.zeros_like(B))
    assert dA[0, 0, 0, 0] == 1.0 and dB[0, 0, 0, 0] == 1.0


def test_relu_backward_closed_form(oracle):
    x = np.array([-1.0, -0.0, 0.0, 1e-30, 2.0, np.nan, np.inf, -np.inf], np.float32)
    dy = np.arange(1, 9, dtype=np.float32)
    got = oracle.relu_backward(x, dy)
    assert np.array_equal(got, np.array([0, 0, 0, 4, 5, 0, 7, 0], np.float32))


def test_add_backward_copy_and_broadcast_sum(oracle):
    rng = np.random.default_rng(7)
    dout = rng.integers(-5, 6, (3, 2, 4, 5)).astype(np.float32)
    same = oracle.add_backward(np.full(dout.shape, 99, np.float32), dout)
    assert np.array_equal(same, dout)                            # equal shapes: overwritten (memcpy)
    d0 = rng.integers(-5, 6, (1, 2, 4, 5)).astype(np.float32)
    assert np.array_equal(oracle.add_backward(d0, dout), d0 + dout.sum(axis=0, keepdims=True))
    d1 = rng.integers(-5, 6, (1, 1, 4, 5)).astype(np.float32)
    assert np.array_equal(oracle.add_backward(d1, dout), d1 + dout.sum(axis=(0, 1), keepdims=True))


@pytest.mark.parametrize("shape,k_h,k_w,stride,pad", [((2, 3, 4, 5), 3, 3, 1, 1), ((1, 2, 7, 6), 3, 2, 2, 0),
                                                      ((2, 1, 5, 5), 5, 5, 1, 2), ((1, 3, 8, 9), 2, 4, 2, 2)])
def test_im2col_backward_loop_nest_and_adjoint(oracle, shape, k_h, k_w, stride, pad):
    # test/Test.cpp:3011-3072 loop nest (first case is the reference's own configuration)
    n, c, h, w = shape
    H_out, W_out = (h + 2 * pad - k_h) // stride + 1, (w + 2 * pad - k_w) // stride + 1
    rng = np.random.default_rng(11)
    grad = rng.integers(1, 10, n * H_out * W_out * k_h * k_w * c).astype(np.float32)
    want = np.zeros(n * c * h * w, np.float32)
    for b in range(n):
        for i in range(H_out):
            for j in range(W_out):
                for r in range(k_h):
                    for s in range(k_w):
                        for ci in range(c):
                            h_in, w_in = i * stride - pad + r, j * stride - pad + s
                            if 0 <= h_in < h and 0 <= w_in < w:
                                want[b * c * h * w + ci * h * w + h_in * w + w_in] += grad[
                                    b * (H_out * W_out * k_h * k_w * c) + (i * W_out + j) * (k_h * k_w * c) + ci * k_h * k_w + r * k_w + s]
    got = oracle.im2col_backward(np.zeros(shape, np.float32), grad, k_h, k_w, stride, pad)
    assert np.array_equal(got.reshape(-1), want)
    # adjoint of the forward gather: <im2col(x), g> == <x, im2col_backward(g)>
    x = rng.integers(-4, 5, shape).astype(np.float32)
    assert float((oracle.im2col(x, k_h, k_w, stride, pad).reshape(-1).astype(np.float64) * grad).sum()) == \
        float((x.reshape(-1).astype(np.float64) * got.reshape(-1)).sum())
    # accumulates onto what the gradient already holds
    again = oracle.im2col_backward(got, grad, k_h, k_w, stride, pad)
    assert np.array_equal(again, 2 * got)


def test_col2im_backward_loop_nest_and_inverse(oracle):
    # test/Test.cpp:3144-3177
    n, c, h, w = 2, 3, 4, 5
    rng = np.random.default_rng(13)
    inp = rng.random(n * c * h * w).astype(np.float32)
    exp = np.empty_like(inp)
    for i in range(n):
        for j in range(c):
            for k in range(h):
                for l in range(w):
                    exp[i * c * h * w + j * h * w + k * w + l] = inp[i * c * h * w + (k * w + l) * c + j]
    got = oracle.col2im_backward(exp.reshape(n, c, h, w))
    assert np.array_equal(got.reshape(-1), inp)
    assert np.array_equal(oracle.col2im(got, h, w).reshape(-1), exp)   # inverse of the forward transpose


@pytest.mark.parametrize("N,C,H,W,O,K,stride,pad,wb", [(2, 3, 7, 8, 4, 3, 2, 1, 1), (1, 2, 9, 9, 3, 3, 2, 0, 1), (2, 2, 11, 10, 2, 5, 3, 2, 2),
                                                        (1, 3, 8, 6, 2, 1, 2, 0, 1), (2, 3, 10, 12, 3, 3, 4, 1, 1), (1, 2, 7, 7, 2, 2, 2, 1, 1)])
def test_strided_conv2d_backward_data_equals_the_pinned_chain(oracle, N, C, H, W, O, K, stride, pad, wb):
    # the strided form of the statement below against the same chain (Img2Col.backward takes the stride), including
    # input rows and columns the strided windows never reach (their gradient stays what it was), and the adjoint identity
    rng = np.random.default_rng(N + 10 * C + 100 * H + O + 7 * stride)
    Ho, Wo = (H + 2 * pad - K) // stride + 1, (W + 2 * pad - K) // stride + 1
    dy = rng.integers(-4, 5, size=(N, O, Ho, Wo)).astype(np.float32)
    w = rng.integers(-4, 5, size=(wb, 1, C * K * K, O)).astype(np.float32)
    dx0 = rng.integers(-3, 4, size=(N, C, H, W)).astype(np.float32)
    got = oracle.conv2d_backward_data(dx0.copy(), dy, w, K, K, pad, stride)
    col = np.zeros((N, 1, Ho * Wo, C * K * K), np.float32)
    dcol, _ = oracle.matmul_backward(col, w, oracle.col2im_backward(dy), dA0=np.zeros_like(col))
    assert np.array_equal(got, oracle.im2col_backward(dx0, dcol, K, K, stride, pad))
    x = rng.integers(-4, 5, size=(N, C, H, W)).astype(np.float32)
    y = oracle.col2im(oracle.tensorcore_gemm(oracle.im2col(x, K, K, stride, pad), w), Ho, Wo)
    assert float((y.astype(np.float64) * dy).sum()) == float((x.astype(np.float64) * (got - dx0)).sum())


@pytest.mark.parametrize("N,C,H,W,O,K,pad,wb", [(2, 3, 5, 6, 4, 3, 1, 1), (1, 2, 4, 4, 3, 3, 0, 1), (2, 2, 6, 5, 2, 3, 2, 2),
                                                 (1, 3, 5, 5, 2, 1, 0, 1), (3, 4, 7, 9, 5, 3, 1, 3)])
def test_conv2d_backward_data_equals_the_pinned_chain(oracle, N, C, H, W, O, K, pad, wb):
    # the one-statement data gradient == Col2Img.backward -> MatMul.backward (dA) -> Img2Col.backward, each of
    # which is pinned above; exact on integers, and the adjoint of the forward convolution
    rng = np.random.default_rng(N + 10 * C + 100 * H + O)
    Ho, Wo = H + 2 * pad - K + 1, W + 2 * pad - K + 1
    dy = rng.integers(-4, 5, size=(N, O, Ho, Wo)).astype(np.float32)
    w = rng.integers(-4, 5, size=(wb, 1, C * K * K, O)).astype(np.float32)
    dx0 = rng.integers(-3, 4, size=(N, C, H, W)).astype(np.float32)
    got = oracle.conv2d_backward_data(dx0.copy(), dy, w, K, K, pad)
    col = np.zeros((N, 1, Ho * Wo, C * K * K), np.float32)
    dcol, _ = oracle.matmul_backward(col, w, oracle.col2im_backward(dy), dA0=np.zeros_like(col))
    assert np.array_equal(got, oracle.im2col_backward(dx0, dcol, K, K, 1, pad))
    x = rng.integers(-4, 5, size=(N, C, H, W)).astype(np.float32)
    y = oracle.col2im(oracle.tensorcore_gemm(oracle.im2col(x, K, K, 1, pad), w), Ho, Wo)
    assert float((y.astype(np.float64) * dy).sum()) == float((x.astype(np.float64) * (got - dx0)).sum())


@pytest.mark.parametrize("N,C,H,W,O,K,pad,wb", [(2, 3, 5, 6, 4, 3, 1, 1), (1, 2, 4, 4, 3, 3, 0, 1), (2, 2, 6, 5, 2, 3, 2, 2),
                                                 (1, 3, 5, 5, 2, 1, 0, 1), (3, 4, 7, 9, 5, 3, 1, 3)])
def test_conv2d_backward_weights_equals_the_pinned_chain(oracle, N, C, H, W, O, K, pad, wb):
    # the one-statement weight gradient == Img2Col.forward -> MatMul.backward (dB) fed by Col2Img.backward;
    # exact on integers
    rng = np.random.default_rng(N + 10 * C + 100 * H + O + 7)
    Ho, Wo = H + 2 * pad - K + 1, W + 2 * pad - K + 1
    x = rng.integers(-4, 5, size=(N, C, H, W)).astype(np.float32)
    dy = rng.integers(-4, 5, size=(N, O, Ho, Wo)).astype(np.float32)
    dw0 = rng.integers(-3, 4, size=(wb, 1, C * K * K, O)).astype(np.float32)
    got = oracle.conv2d_backward_weights(dw0.copy(), x, dy, K, K, pad)
    _, want = oracle.matmul_backward(oracle.im2col(x, K, K, 1, pad), dw0, oracle.col2im_backward(dy), dB0=dw0)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("N,C,H,W,O,Kh,Kw,stride,pad,wb", [(2, 3, 9, 8, 4, 3, 3, 2, 1, 1), (1, 2, 11, 13, 3, 5, 5, 1, 2, 1),
                                                            (2, 2, 10, 9, 2, 5, 3, 2, 0, 2), (1, 3, 12, 12, 2, 7, 7, 3, 3, 1),
                                                            (3, 1, 6, 7, 5, 2, 4, 1, 1, 3)])
def test_strided_conv2d_backward_weights_equals_the_pinned_chain(oracle, N, C, H, W, O, Kh, Kw, stride, pad, wb):
    # any kernel extent and stride: the one-statement gradient == Img2Col.forward (whose index formula carries the
    # stride) -> MatMul.backward (dB); exact on integers, so a wrong stride, tap or padding term shows
    rng = np.random.default_rng(N + 10 * C + 100 * H + O + 7 * stride + Kh)
    Ho, Wo = (H + 2 * pad - Kh) // stride + 1, (W + 2 * pad - Kw) // stride + 1
    x = rng.integers(-4, 5, size=(N, C, H, W)).astype(np.float32)
    dy = rng.integers(-4, 5, size=(N, O, Ho, Wo)).astype(np.float32)
    dw0 = rng.integers(-3, 4, size=(wb, 1, C * Kh * Kw, O)).astype(np.float32)
    got = oracle.conv2d_backward_weights(dw0.copy(), x, dy, Kh, Kw, pad, stride)
    _, want = oracle.matmul_backward(oracle.im2col(x, Kh, Kw, stride, pad), dw0, oracle.col2im_backward(dy), dB0=dw0)
    assert np.array_equal(got, want)
