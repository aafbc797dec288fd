"""Parity of the backward entry points (GEMM backward with batch reduction, MatMul / Add / ReLU /
im2col / col2im backward) on the GPU with the CPU oracle, through the C-ABI.  Integer-valued cases
must match bit for bit (sums are exact in any order); float cases meet max-rel <= 1e-3 /
Frobenius-rel <= 1e-4 against fp64 accumulation of the same fp16-rounded operands (max-rel floored
at the RMS of the truth)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

MAX_REL, FROB_REL = 1e-3, 1e-4


@pytest.fixture(scope="module")
def nz():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from neuzephyr_amd import capi
    capi.load()
    return capi


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()


def host(t):
    return t.cpu().numpy()


def check_tolerance(oracle, got, truth64, tag=""):
    rms = float(np.sqrt(np.mean(np.square(truth64)))) or 1.0
    mr, fr = oracle.errors(got, truth64, rms)
    assert mr <= MAX_REL and fr <= FROB_REL, f"{tag}: max_rel {mr:.3e} frob_rel {fr:.3e}"


def ints(rng, shape, lo=-4, hi=5):
    return rng.integers(lo, hi, shape).astype(np.float32)


def test_matmul_backward_reference_vectors(nz):
    # test/Test.cpp:820-903
    n, c, m, k, p = 2, 3, 2, 3, 2
    A = np.ones((n, 1, m, k), np.float32); B = np.ones((1, c, k, p), np.float32); dC = np.ones((n, c, m, p), np.float32)
    dA, dB = dev(np.zeros_like(A)), dev(np.zeros_like(B))
    nz.matmul_backward(dA, dB, dev(A), dev(B), dev(dC))
    assert np.array_equal(host(dA), np.full_like(A, 2 * c)) and np.array_equal(host(dB), np.full_like(B, 2 * n))
    A = np.array([1, 2, 3, 4, 5, 6, 2, 3, 4, 5, 6, 7, 3, 4, 5, 6, 7, 8] * 2, np.float32).reshape(n, c, m, k)
    B = np.array([1, 4, 2, 5, 3, 6, 2, 5, 3, 6, 4, 7, 3, 6, 4, 7, 5, 8], np.float32).reshape(1, c, k, p)
    Agrad = np.array([5, 7, 9, 5, 7, 9, 7, 9, 11, 7, 9, 11, 9, 11, 13, 9, 11, 13] * 2, np.float32).reshape(n, c, m, k)
    Bgrad = np.array([10, 10, 14, 14, 18, 18, 14, 14, 18, 18, 22, 22, 18, 18, 22, 22, 26, 26], np.float32).reshape(1, c, k, p)
    dA, dB = dev(np.zeros_like(A)), dev(np.zeros_like(B))
    nz.matmul_backward(dA, dB, dev(A), dev(B), dev(dC))
    assert np.array_equal(host(dA), Agrad) and np.array_equal(host(dB), Bgrad)


# (shapeA, shapeB): every broadcast pattern, ragged extents, the vector collapses and the K-folded reductions
MATMUL_BWD_CASES = [
    ((2, 3, 5, 7), (2, 3, 7, 6)),        # no broadcast
    ((2, 1, 5, 7), (1, 3, 7, 6)),        # both broadcast in different dims
    ((1, 1, 9, 4), (3, 2, 4, 5)),        # A shared: dA reduces over n and c (sequential members)
    ((3, 2, 9, 4), (1, 1, 4, 5)),        # B shared: dB reduces over both, folded into K
    ((4, 1, 33, 20), (1, 1, 20, 17)),    # conv-like: column matrix per image, shared weights
    ((1, 1, 24, 16), (5, 1, 16, 1)),     # Model::Linear: W[OUT,IN] * x_n[IN,1]
    ((6, 1, 1, 12), (1, 1, 12, 10)),     # row vectors against a shared matrix
    ((1, 3, 8, 8), (4, 3, 8, 8)),        # reduce over n only, c stays a batch
    ((2, 2, 1, 1), (2, 2, 1, 1)),
    ((1, 1, 130, 70), (1, 1, 70, 140)),  # one matrix, larger than a tile
]


@pytest.mark.parametrize("sa,sb", MATMUL_BWD_CASES)
def test_matmul_backward_integers_bit_exact(nz, oracle, sa, sb):
    rng = np.random.default_rng(hash((sa, sb)) % (1 << 31))
    A, B = ints(rng, sa, -3, 4), ints(rng, sb, -3, 4)
    sc = (max(sa[0], sb[0]), max(sa[1], sb[1]), sa[2], sb[3])
    dC = ints(rng, sc, -3, 4)
    dA0, dB0 = ints(rng, sa, -9, 10), ints(rng, sb, -9, 10)       # gradients already hold something: "+="
    want_dA, want_dB = oracle.matmul_backward(A, B, dC, dA0, dB0)
    dA, dB = dev(dA0), dev(dB0)
    nz.matmul_backward(dA, dB, dev(A), dev(B), dev(dC))
    assert np.array_equal(host(dA), want_dA), "dA"
    assert np.array_equal(host(dB), want_dB), "dB"
    # one gradient at a time
    dA = dev(dA0); nz.matmul_backward(dA, None, dev(A), dev(B), dev(dC)); assert np.array_equal(host(dA), want_dA)
    dB = dev(dB0); nz.matmul_backward(None, dB, dev(A), dev(B), dev(dC)); assert np.array_equal(host(dB), want_dB)


@pytest.mark.parametrize("sa,sb,sc", [((2, 3, 5, 7), (2, 3, 7, 6), (2, 3, 5, 6)), ((3, 1, 5, 7), (1, 2, 7, 6), (1, 1, 5, 6)),
                                     ((3, 2, 5, 7), (3, 2, 7, 6), (1, 2, 5, 6)), ((3, 2, 5, 7), (3, 2, 7, 6), (3, 1, 5, 6)),
                                     ((1, 1, 40, 33), (1, 1, 33, 50), (1, 1, 40, 50))])
def test_gemm_backward_entry_integers_bit_exact(nz, oracle, sa, sb, sc):
    rng = np.random.default_rng(17)
    A, B, C0 = ints(rng, sa), ints(rng, sb), ints(rng, sc, -9, 10)
    want = oracle.gemm_backward(A, B, C0)
    C = dev(C0)
    nz.gemm_backward(dev(A), dev(B), C)
    assert np.array_equal(host(C), want)


def test_linear_layer_backward_float_tolerance(nz, oracle):
    # Model::Linear shapes (W[1,1,OUT,IN] * x[n,1,IN,1]) at a size the oracle finishes quickly
    n, IN, OUT = 192, 256, 320
    W = oracle.fill((1, 1, OUT, IN), 2101, "uniform", -0.0765, 0.0765)
    x = oracle.fill((n, 1, IN, 1), 2102, "normal", 0.0, 1.0)
    dy = oracle.fill((n, 1, OUT, 1), 2103, "normal", 0.0, 1.0)
    dW, dx = dev(np.zeros_like(W)), dev(np.zeros_like(x))
    nz.matmul_backward(dW, dx, dev(W), dev(x), dev(dy))
    dyr, xr, Wr = (oracle.round_f16(t).astype(np.float64) for t in (dy, x, W))
    truth_dW = dyr.reshape(n, OUT).T @ xr.reshape(n, IN)
    truth_dx = dyr.reshape(n, OUT) @ Wr.reshape(OUT, IN)
    check_tolerance(oracle, host(dW).reshape(OUT, IN), truth_dW, "dW")
    check_tolerance(oracle, host(dx).reshape(n, IN), truth_dx, "dx")


def test_conv_weight_gradient_float_tolerance(nz, oracle):
    # dW = sum over images of col_n^T * dZ_n : the reduction folded into one contraction of length n * pixels
    n, P, CKK, O = 6, 400, 72, 40
    col = oracle.fill((n, 1, P, CKK), 2201, "normal", 0.0, 1.0)
    Wt = oracle.fill((1, 1, CKK, O), 2202, "normal", 0.0, 0.1)
    dZ = oracle.fill((n, 1, P, O), 2203, "normal", 0.0, 1.0)
    dcol, dW = dev(np.zeros_like(col)), dev(np.zeros_like(Wt))
    nz.matmul_backward(dcol, dW, dev(col), dev(Wt), dev(dZ))
    cr, wr, zr = (oracle.round_f16(t).astype(np.float64) for t in (col, Wt, dZ))
    truth_dW = cr.reshape(n * P, CKK).T @ zr.reshape(n * P, O)
    truth_dcol = zr.reshape(n * P, O) @ wr.reshape(CKK, O).T
    check_tolerance(oracle, host(dW).reshape(CKK, O), truth_dW, "dW")
    check_tolerance(oracle, host(dcol).reshape(n * P, CKK), truth_dcol, "dcol")


def test_relu_backward_bit_exact(nz, oracle):
    rng = np.random.default_rng(23)
    for n in (1, 3, 4, 255, 4099):
        x = rng.standard_normal(n).astype(np.float32)
        x[:: 7] = 0.0
        if n > 8:
            x[1], x[2], x[3], x[5] = np.nan, -0.0, np.inf, -np.inf
        dy = rng.standard_normal(n).astype(np.float32)
        assert np.array_equal(host(nz.relu_backward(dev(x), dev(dy))), oracle.relu_backward(x, dy))


def test_add_backward_bit_exact(nz, oracle):
    rng = np.random.default_rng(29)
    for s_in, s_out in [((3, 2, 4, 5), (3, 2, 4, 5)), ((1, 2, 4, 5), (3, 2, 4, 5)), ((3, 1, 4, 5), (3, 2, 4, 5)),
                        ((1, 1, 30, 7), (4, 3, 30, 7)), ((1, 1, 64, 1), (5, 1, 64, 1))]:
        din0, dout = ints(rng, s_in, -9, 10), ints(rng, s_out, -9, 10)
        got = nz.add_backward(dev(din0), dev(dout))
        assert np.array_equal(host(got), oracle.add_backward(din0, dout)), (s_in, s_out)
    # float data: same summation order as the oracle -> identical bits
    din0 = rng.standard_normal((1, 2, 9, 5)).astype(np.float32)
    dout = rng.standard_normal((7, 2, 9, 5)).astype(np.float32)
    assert np.array_equal(host(nz.add_backward(dev(din0), dev(dout))), oracle.add_backward(din0, dout))
    with pytest.raises(nz.NzHipError):
        nz.add_backward(dev(np.zeros((2, 1, 3, 3))), dev(np.zeros((3, 1, 3, 3))))


def test_add_backward_with_hundreds_of_members_per_element(nz, oracle):
    # a Linear layer's bias against a batch of thousands: the members are added in chunks (fixed order, not the single
    # ascending chain of the oracle): exact on integers, a few ulp on floats, the same bits on every run
    rng = np.random.default_rng(31)
    for s_in, s_out in [((1, 1, 300, 1), (1000, 1, 300, 1)), ((1, 1, 50, 3), (20, 9, 50, 3)), ((1, 3, 70, 1), (400, 3, 70, 1)),
                        ((2, 1, 33, 2), (2, 130, 33, 2))]:
        din0, dout = ints(rng, s_in, -9, 10), ints(rng, s_out, -9, 10)
        assert np.array_equal(host(nz.add_backward(dev(din0), dev(dout))), oracle.add_backward(din0, dout)), (s_in, s_out)
    din0 = rng.standard_normal((1, 1, 300, 1)).astype(np.float32)
    dout = rng.standard_normal((1000, 1, 300, 1)).astype(np.float32)
    a = host(nz.add_backward(dev(din0), dev(dout)))
    b = host(nz.add_backward(dev(din0), dev(dout)))
    assert np.array_equal(a, b)
    truth = din0.astype(np.float64) + dout.astype(np.float64).sum(axis=0, keepdims=True)
    assert np.abs(a - truth).max() <= 1e-5 * np.abs(dout).sum(axis=0).max()


def test_fill_writes_every_element(nz):
    import torch
    for n in (1, 3, 4, 1023, 4096, 100003):
        t = torch.full((n + 9,), 7.0, device="cuda")
        nz.fill(t[4:4 + n], -2.5)                      # 16-byte aligned start
        want = np.full(n + 9, 7.0, np.float32); want[4:4 + n] = -2.5
        assert np.array_equal(host(t), want)
        t = torch.full((n + 9,), 7.0, device="cuda")
        nz.fill(t[1:1 + n], 0.125)                     # unaligned start
        want = np.full(n + 9, 7.0, np.float32); want[1:1 + n] = 0.125
        assert np.array_equal(host(t), want)


IM2COL_CASES = [((2, 3, 4, 5), 3, 3, 1, 1), ((1, 1, 1, 1), 1, 1, 1, 0), ((2, 2, 7, 6), 3, 2, 2, 0),
                ((1, 3, 8, 9), 2, 4, 2, 2), ((3, 1, 5, 5), 5, 5, 1, 2), ((2, 4, 6, 6), 1, 1, 3, 0),
                ((2, 5, 33, 47), 3, 3, 1, 1), ((1, 2, 9, 9), 3, 3, 3, 1),
                # wide rows and many channels, strides 2 and 4, padding beyond the reach of a tap, a window of most of the image
                ((2, 19, 12, 70), 3, 3, 1, 1), ((1, 6, 10, 150), 5, 5, 1, 2), ((1, 3, 11, 300), 7, 7, 2, 3), ((2, 2, 9, 40), 11, 11, 4, 5),
                ((1, 9, 20, 33), 3, 3, 2, 1), ((1, 1, 70, 70), 65, 65, 1, 0)]


@pytest.mark.parametrize("shape,k_h,k_w,stride,pad", IM2COL_CASES)
def test_im2col_backward_bit_exact(nz, oracle, shape, k_h, k_w, stride, pad):
    rng = np.random.default_rng(31)
    n, c, h, w = shape
    Ho, Wo = (h + 2 * pad - k_h) // stride + 1, (w + 2 * pad - k_w) // stride + 1
    dcol = ints(rng, (n, 1, Ho * Wo, c * k_h * k_w), -5, 6)
    dx0 = ints(rng, shape, -9, 10)
    got = nz.im2col_backward(dev(dx0), dev(dcol), k_h, k_w, stride, pad)
    assert np.array_equal(host(got), oracle.im2col_backward(dx0, dcol, k_h, k_w, stride, pad))
    # float data: the gather adds in the oracle's element order -> identical bits
    dcol_f = rng.standard_normal(dcol.shape).astype(np.float32)
    got = nz.im2col_backward(dev(np.zeros(shape, np.float32)), dev(dcol_f), k_h, k_w, stride, pad)
    assert np.array_equal(host(got), oracle.im2col_backward(np.zeros(shape, np.float32), dcol_f, k_h, k_w, stride, pad))


@pytest.mark.parametrize("n,c,h,w", [(2, 3, 4, 5), (1, 1, 1, 1), (3, 40, 9, 11), (2, 128, 16, 16), (1, 1, 50, 70), (3, 7, 1, 1)])
def test_col2im_backward_bit_exact(nz, oracle, n, c, h, w):
    rng = np.random.default_rng(37)
    dy = rng.standard_normal((n, c, h, w)).astype(np.float32)
    got = host(nz.col2im_backward(dev(dy)))
    assert np.array_equal(got, oracle.col2im_backward(dy))
    assert np.array_equal(host(nz.col2im(dev(got), h, w)), dy)       # round trip with the forward transpose


CONV_BWD_DATA = [  # N, C, H, W, O, K, pad, w_batch
    (2, 3, 5, 6, 4, 3, 1, 1), (1, 2, 4, 4, 3, 3, 0, 1), (2, 2, 6, 5, 2, 3, 2, 2), (1, 3, 5, 5, 2, 1, 0, 1),
    (2, 16, 20, 36, 24, 3, 1, 1), (1, 64, 32, 64, 128, 3, 1, 1), (3, 8, 17, 33, 70, 3, 1, 3), (2, 40, 9, 70, 12, 1, 0, 1),
    (1, 3, 40, 40, 1, 3, 1, 1), (2, 1, 12, 16, 2, 3, 1, 1),
    (3, 20, 9, 10, 33, 1, 0, 3), (4, 256, 14, 14, 300, 1, 0, 1),            # 1x1: one batched product (per-sample weights; many channels)
    (4, 300, 14, 14, 64, 3, 1, 1), (16, 256, 7, 7, 40, 3, 1, 1), (2, 96, 28, 28, 160, 3, 1, 1),   # deep layers on small images: accumulation in place on the any-geometry kernel, or through a temporary
    (3, 80, 6, 6, 20, 3, 1, 3), (4, 130, 5, 7, 33, 5, 2, 4),            # per-sample weights larger than the column gradient: the chain on dy as it lies (planes of 36 and 35 pixels)
    (16, 64, 7, 7, 64, 3, 1, 1), (5, 70, 4, 4, 90, 3, 1, 1)]             # tiny images, shared weights: the chain with all images as rows of one product


@pytest.mark.parametrize("N,C,H,W,O,K,pad,wb", CONV_BWD_DATA)
@pytest.mark.parametrize("accumulate", [True, False])
def test_conv2d_backward_data_matches_the_chain_on_integers(nz, oracle, N, C, H, W, O, K, pad, wb, accumulate):
    # one fused call == Col2Img.backward -> MatMul.backward (dA) -> Img2Col.backward, exact on integers
    rng = np.random.default_rng(N * 131 + C * 17 + H * 7 + W + O * 3 + K)
    Ho, Wo = H + 2 * pad - K + 1, W + 2 * pad - K + 1
    dy = rng.integers(-4, 5, size=(N, O, Ho, Wo)).astype(np.float32)
    w = rng.integers(-4, 5, size=(wb, 1, C * K * K, O)).astype(np.float32)
    dx0 = rng.integers(-3, 4, size=(N, C, H, W)).astype(np.float32)
    expect = oracle.conv2d_backward_data(dx0.copy() if accumulate else np.zeros_like(dx0), dy, w, K, K, pad)
    got = host(nz.conv2d_backward_data(dev(dx0), dev(dy), dev(w), K, K, 1, pad, accumulate=accumulate))
    assert np.array_equal(got, expect)


def test_conv2d_backward_data_float_tolerance_and_adjoint(nz, oracle):
    N, C, H, W, O, K, pad = 2, 32, 24, 40, 48, 3, 1
    rng = np.random.default_rng(5)
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    dy = rng.standard_normal((N, O, H, W)).astype(np.float32)
    w = (rng.standard_normal((1, 1, C * K * K, O)) * 0.1).astype(np.float32)
    got = host(nz.conv2d_backward_data(dev(np.zeros_like(x)), dev(dy), dev(w), K, K, 1, pad, accumulate=True))
    # truth: fp64 accumulation over the fp16-rounded operands, tap by tap
    dyr, wr = oracle.round_f16(dy).astype(np.float64), oracle.round_f16(w).astype(np.float64)
    wt = wr[0, 0].reshape(C, K, K, O)
    truth = np.zeros((N, C, H, W))
    for r in range(K):
        for sx in range(K):
            g = np.einsum("nohw,co->nchw", dyr, wt[:, r, sx, :])      # contribution of dy[ho, wo] to x[ho - pad + r, wo - pad + sx]
            h0, w0 = r - pad, sx - pad
            hs, ws = slice(max(0, -h0), min(H, H - h0)), slice(max(0, -w0), min(W, W - w0))
            hd, wd = slice(hs.start + h0, hs.stop + h0), slice(ws.start + w0, ws.stop + w0)
            truth[:, :, hd, wd] += g[:, :, hs, ws]
    rms = float(np.sqrt(np.mean(truth ** 2)))
    mr, fr = oracle.errors(got, truth, rms)
    assert mr <= 1e-3 and fr <= 1e-4, (mr, fr)
    # adjoint identity with the forward kernel: <conv(x), dy> == <x, conv^T(dy)> for rounded x
    xr = oracle.round_f16(x)
    y = host(nz.conv2d_forward(dev(xr), dev(w), None, K, K, 1, pad))
    lhs = float(np.sum(y.astype(np.float64) * dyr))
    rhs = float(np.sum(xr.astype(np.float64) * got.astype(np.float64)))
    assert abs(lhs - rhs) <= 1e-4 * max(abs(lhs), abs(rhs), 1.0)


CONV_BWD_DATA_STRIDED = [  # N, C, H, W, O, K, stride, pad, w_batch: rows and columns no window reaches, strides 2..4, per-sample weights
    (2, 3, 7, 8, 4, 3, 2, 1, 1), (1, 2, 9, 9, 3, 3, 2, 0, 1), (2, 2, 11, 10, 2, 5, 3, 2, 2), (1, 3, 8, 6, 2, 1, 2, 0, 1),
    (2, 16, 21, 36, 24, 3, 2, 1, 1), (1, 64, 32, 64, 128, 3, 2, 1, 1), (3, 8, 17, 33, 70, 5, 2, 2, 3), (2, 24, 30, 40, 16, 3, 4, 1, 1),
    (8, 32, 28, 28, 64, 3, 2, 1, 1),
    # 1x1 with a stride: the gradient on the gathered pixels, put back between pixels that get none
    (2, 20, 9, 11, 33, 1, 2, 0, 1), (3, 130, 7, 13, 24, 1, 3, 0, 3), (4, 256, 14, 14, 64, 1, 2, 0, 1)]


@pytest.mark.parametrize("N,C,H,W,O,K,stride,pad,wb", CONV_BWD_DATA_STRIDED)
@pytest.mark.parametrize("accumulate", [True, False])
def test_strided_conv2d_backward_data_is_exact_on_integers(nz, oracle, N, C, H, W, O, K, stride, pad, wb, accumulate):
    rng = np.random.default_rng(N * 131 + C * 17 + H * 7 + W + O * 3 + K + stride)
    Ho, Wo = (H + 2 * pad - K) // stride + 1, (W + 2 * pad - K) // stride + 1
    dy = rng.integers(-4, 5, size=(N, O, Ho, Wo)).astype(np.float32)
    w = rng.integers(-4, 5, size=(wb, 1, C * K * K, O)).astype(np.float32)
    dx0 = rng.integers(-3, 4, size=(N, C, H, W)).astype(np.float32)
    expect = oracle.conv2d_backward_data(dx0.copy() if accumulate else np.zeros_like(dx0), dy, w, K, K, pad, stride)
    got = host(nz.conv2d_backward_data(dev(dx0), dev(dy), dev(w), K, K, stride, pad, accumulate=accumulate))
    assert np.array_equal(got, expect)


def test_conv2d_backward_data_rejects_what_it_does_not_cover(nz):
    from neuzephyr_amd.capi import NzHipError
    dx, dy, w = dev(np.zeros((1, 2, 8, 8))), dev(np.zeros((1, 3, 7, 3))), dev(np.zeros((1, 1, 2 * 2 * 6, 3)))
    with pytest.raises(NzHipError):
        nz.conv2d_backward_data(dx, dy, w, 2, 6, 1, 0)              # a kernel that is not square
    dx, dy, w = dev(np.zeros((1, 2, 40, 40))), dev(np.zeros((1, 3, 5, 5))), dev(np.zeros((1, 1, 18, 3)))
    with pytest.raises(NzHipError):
        nz.conv2d_backward_data(dx, dy, w, 3, 3, 9, 1)              # stride above 8


CONV_BWD_W = [  # N, C, H, W, O, w_batch   (3x3, stride 1, pad 1; W a multiple of 8 takes 16-byte loads)
    (1, 3, 4, 8, 2, 1), (2, 5, 7, 16, 9, 1), (2, 32, 9, 24, 40, 2), (3, 40, 6, 136, 130, 1), (1, 64, 16, 128, 128, 1),
    (2, 33, 5, 264, 129, 2), (4, 8, 33, 40, 16, 1), (1, 1, 1, 8, 1, 1),
    (2, 3, 28, 28, 6, 1), (1, 5, 7, 9, 4, 1), (2, 20, 6, 131, 33, 2), (1, 2, 3, 1, 2, 1), (1, 4, 5, 127, 3, 1),
    # C <= 4, O <= 2, W a multiple of 4: the streaming kernel (strips of 16 rows, 256 columns per wave; partial last
    # strip, several column blocks with a ragged last one, per-sample and shared weights)
    (2, 3, 20, 24, 1, 2), (3, 1, 33, 260, 1, 3), (1, 4, 5, 8, 2, 1), (2, 2, 70, 516, 2, 1), (2, 3, 64, 256, 1, 1),
    (1, 1, 1, 4, 1, 1),
    # 128 or more input channels on images up to 64 wide: the gather kernel although the rows are multiples of 8 wide
    (2, 130, 9, 24, 40, 1), (2, 128, 6, 64, 33, 2)]


@pytest.mark.parametrize("N,C,H,W,O,wb", CONV_BWD_W)
def test_conv2d_backward_weights_is_bit_exact_on_integers(nz, oracle, N, C, H, W, O, wb):
    # one fused call == Img2Col.forward -> MatMul.backward (dB); every partial sum is an exact integer
    rng = np.random.default_rng(N * 131 + C * 17 + H * 7 + W + O * 3 + wb)
    x = rng.integers(-3, 4, size=(N, C, H, W)).astype(np.float32)
    dy = rng.integers(-3, 4, size=(N, O, H, W)).astype(np.float32)
    dw0 = rng.integers(-5, 6, size=(wb, 1, C * 9, O)).astype(np.float32)
    expect = oracle.conv2d_backward_weights(dw0.copy(), x, dy, 3, 3, 1)
    got = host(nz.conv2d_backward_weights(dev(dw0), dev(x), dev(dy), 3, 3, 1, 1))
    assert np.array_equal(got, expect)


def _conv_grad_sweep_cases(seed, count):
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        C = int(rng.choice([1, 2, 3, 4, 8, 17, 32, 40, 64, 70, 128]))
        O = int(rng.choice([1, 2, 5, 33, 64, 100, 128, 130]))
        H = int(rng.integers(1, 20))
        W = int(rng.choice([int(rng.integers(1, 40)), 8, 24, 64, 68, 72, 128, 136, 260]))
        N = int(rng.integers(1, 4))
        wb = int(rng.choice([1, 1, N]))
        if N * O * H * W * C * 9 > 3e8:
            continue
        cases.append((N, C, H, W, O, wb))
    return cases


@pytest.mark.parametrize("N,C,H,W,O,wb", _conv_grad_sweep_cases(20252, 48))
def test_conv2d_gradients_random_sweep_integers_bit_exact(nz, oracle, N, C, H, W, O, wb):
    # 3x3, stride 1, padding 1 (what the fused gradients cover): both gradients against the node chain's sums
    rng = np.random.default_rng(N * 5 + C * 7 + H * 11 + W * 13 + O * 17 + wb)
    x = rng.integers(-3, 4, size=(N, C, H, W)).astype(np.float32)
    dy = rng.integers(-3, 4, size=(N, O, H, W)).astype(np.float32)
    w = rng.integers(-3, 4, size=(wb, 1, C * 9, O)).astype(np.float32)
    dw0 = rng.integers(-5, 6, size=(wb, 1, C * 9, O)).astype(np.float32)
    expect_dw = oracle.conv2d_backward_weights(dw0.copy(), x, dy, 3, 3, 1)
    got_dw = host(nz.conv2d_backward_weights(dev(dw0), dev(x), dev(dy), 3, 3, 1, 1))
    assert np.array_equal(got_dw, expect_dw)
    dx0 = rng.integers(-3, 4, size=(N, C, H, W)).astype(np.float32)
    expect_dx = oracle.conv2d_backward_data(dx0.copy(), dy, w, 3, 3, 1)
    got_dx = host(nz.conv2d_backward_data(dev(dx0), dev(dy), dev(w), 3, 3, 1, 1, accumulate=True))
    assert np.array_equal(got_dx, expect_dx)


CONV1X1_BWD_W = [  # N, C, H, W, O, w_batch   (1x1, stride 1, no padding: one batched product, no column matrix)
    (1, 1, 1, 1, 1, 1), (1, 3, 4, 5, 2, 1), (2, 5, 7, 9, 6, 1), (3, 16, 8, 8, 24, 3), (2, 64, 16, 16, 128, 1), (4, 70, 9, 11, 33, 1),
    (2, 128, 12, 20, 64, 2), (5, 3, 30, 33, 1, 1), (1, 256, 8, 8, 256, 1), (6, 8, 5, 5, 8, 6),
    # per-sample weights (dw is read and written in place as the product's bias matrix) with a long contraction
    # that is split into chunks, with pixel rows that forbid 16-byte loads (padded copies), and on the two-pass route
    (2, 40, 32, 40, 24, 2), (2, 24, 31, 35, 40, 2), (3, 130, 45, 23, 70, 3), (2, 512, 48, 48, 512, 2)]


@pytest.mark.parametrize("N,C,H,W,O,wb", CONV1X1_BWD_W)
def test_conv1x1_backward_weights_is_bit_exact_on_integers(nz, oracle, N, C, H, W, O, wb):
    rng = np.random.default_rng(N * 31 + C * 17 + H * 7 + W + O * 3 + wb)
    x = rng.integers(-3, 4, size=(N, C, H, W)).astype(np.float32)
    dy = rng.integers(-3, 4, size=(N, O, H, W)).astype(np.float32)
    dw0 = rng.integers(-5, 6, size=(wb, 1, C, O)).astype(np.float32)
    expect = oracle.conv2d_backward_weights(dw0.copy(), x, dy, 1, 1, 0)
    got = host(nz.conv2d_backward_weights(dev(dw0), dev(x), dev(dy), 1, 1, 1, 0))
    assert np.array_equal(got, expect)
    # the node chain's own product gives the same numbers: dB of MatMul.backward with the column matrix of a 1x1 kernel
    col = host(nz.im2col(dev(x), 1, 1, 1, 0))                                     # [N, 1, HW, C]
    dcol = np.ascontiguousarray(dy.reshape(N, 1, O, H * W).transpose(0, 1, 3, 2))  # [N, 1, HW, O]
    chain = dw0.astype(np.float64).copy()
    for n in range(N):
        chain[n if wb > 1 else 0, 0] += col[n, 0].astype(np.float64).T @ dcol[n, 0].astype(np.float64)
    assert np.array_equal(got.astype(np.float64), chain)


CONV_GEN_BWD_W = [  # N, C, H, W, O, Kh, Kw, stride, pad, w_batch: every geometry but 3x3 s1 p1 and 1x1 s1 p0
    (2, 3, 9, 8, 4, 3, 3, 2, 1, 1), (1, 2, 11, 13, 3, 5, 5, 1, 2, 1), (2, 2, 10, 9, 2, 5, 3, 2, 0, 2), (1, 3, 12, 12, 2, 7, 7, 3, 3, 1),
    (3, 1, 6, 7, 5, 2, 4, 1, 1, 3), (2, 20, 16, 300, 70, 5, 5, 1, 2, 1),      # several 128-pixel segments per row, two o tiles, 4 chunks
    (2, 40, 33, 37, 100, 3, 3, 2, 1, 1), (2, 7, 20, 20, 9, 3, 3, 1, 0, 1), (1, 5, 40, 260, 6, 3, 3, 4, 2, 1), (2, 3, 30, 30, 3, 11, 11, 4, 5, 2),
    (1, 130, 12, 12, 8, 1, 1, 2, 0, 1), (2, 6, 40, 50, 5, 3, 3, 1, 0, 1), (1, 4, 70, 64, 130, 5, 5, 1, 2, 1),   # segment widths 64 and (two rows of) 64
    # rows that allow 16-byte loads (the eight-wave kernel): stride 2 with seven pieces of input rows per thread and two chunks,
    # per-sample weights, stride 2 over three segments per row, stride 1 with seven pieces per thread
    (2, 40, 32, 64, 100, 3, 3, 2, 1, 1), (2, 6, 16, 16, 5, 5, 5, 1, 2, 2), (1, 8, 12, 520, 12, 3, 3, 2, 1, 1), (1, 70, 10, 128, 8, 2, 1, 1, 0, 1),
    # many small images: a workgroup walks several images and leaves one set of partial sums for them (rows that are whole
    # 16-byte pieces, and rows that are not); 3x3 stride 1 pad 1 on 28- and 14-wide images, which the gather kernel takes
    # from the kernel built for rows that are multiples of 8 wide
    (40, 256, 8, 8, 16, 3, 3, 2, 1, 1), (40, 256, 8, 8, 16, 3, 3, 1, 0, 1), (3, 40, 28, 28, 24, 3, 3, 1, 1, 1), (20, 200, 14, 14, 20, 3, 3, 1, 1, 1),
    # 1x1 with a stride: the pixels it looks at gathered once, then the 1x1 stride-1 product (shared and per-sample weights)
    (4, 70, 14, 14, 130, 1, 1, 2, 0, 1), (3, 20, 9, 11, 33, 1, 1, 3, 0, 3),
    # shared weights and fewer than 64 output pixels per image: one product over the pixels of all images (3x3 stride 2,
    # 1x1, 3x3 on 4x4 images, 1x1 stride 2); the last has too few pixels in all and stays with the gather kernel
    (16, 128, 14, 14, 128, 3, 3, 2, 1, 1), (8, 300, 7, 7, 260, 1, 1, 1, 0, 1), (70, 64, 4, 4, 128, 3, 3, 1, 1, 1),
    (6, 256, 13, 13, 256, 1, 1, 2, 0, 1), (4, 128, 7, 7, 128, 3, 3, 1, 1, 1)]


@pytest.mark.parametrize("N,C,H,W,O,Kh,Kw,stride,pad,wb", CONV_GEN_BWD_W)
def test_conv_backward_weights_any_geometry_is_bit_exact_on_integers(nz, oracle, N, C, H, W, O, Kh, Kw, stride, pad, wb):
    rng = np.random.default_rng(N * 31 + C * 17 + H * 7 + W + O * 3 + Kh + 5 * stride)
    Ho, Wo = (H + 2 * pad - Kh) // stride + 1, (W + 2 * pad - Kw) // stride + 1
    x = rng.integers(-3, 4, size=(N, C, H, W)).astype(np.float32)
    dy = rng.integers(-3, 4, size=(N, O, Ho, Wo)).astype(np.float32)
    dw0 = rng.integers(-5, 6, size=(wb, 1, C * Kh * Kw, O)).astype(np.float32)
    expect = oracle.conv2d_backward_weights(dw0.copy(), x, dy, Kh, Kw, pad, stride)
    got = host(nz.conv2d_backward_weights(dev(dw0), dev(x), dev(dy), Kh, Kw, stride, pad))
    assert np.array_equal(got, expect)


@pytest.mark.parametrize("N,C,H,W,O,Kh,Kw,stride,pad,wb", [c for c in CONV_GEN_BWD_W if c[3] % 4 != 0 or ((c[3] + 2 * c[8] - c[6]) // c[7] + 1) % 4 != 0] +
                         [(3, 40, 7, 7, 24, 1, 1, 1, 0, 1), (2, 20, 5, 5, 33, 1, 1, 1, 0, 2), (2, 70, 35, 35, 9, 1, 1, 1, 0, 1)])   # and 1x1 products on planes of 49, 25, 1225 pixels
def test_conv_backward_weights_on_rows_widened_to_16_byte_pieces(nz, oracle, monkeypatch, N, C, H, W, O, Kh, Kw, stride, pad, wb):
    # Large layers whose rows of x or dy are not whole 16-byte pieces run on zero-filled copies with rows of the next
    # multiple of 4; the library reads NZHIP_CONV_WIDEN per call, so the copies can be forced for these small shapes.
    monkeypatch.setenv("NZHIP_CONV_WIDEN", "1")
    test_conv_backward_weights_any_geometry_is_bit_exact_on_integers(nz, oracle, N, C, H, W, O, Kh, Kw, stride, pad, wb)


def test_conv_backward_weights_any_geometry_float_tolerance(nz, oracle):
    N, C, H, W, O, K, stride, pad = 2, 24, 40, 72, 48, 5, 2, 2
    Ho, Wo = (H + 2 * pad - K) // stride + 1, (W + 2 * pad - K) // stride + 1
    rng = np.random.default_rng(29)
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    dy = rng.standard_normal((N, O, Ho, Wo)).astype(np.float32)
    got = host(nz.conv2d_backward_weights(dev(np.zeros((1, 1, C * K * K, O))), dev(x), dev(dy), K, K, stride, pad))
    xr = np.pad(oracle.round_f16(x).astype(np.float64), ((0, 0), (0, 0), (pad, pad), (pad, pad)))
    dyr = oracle.round_f16(dy).astype(np.float64)
    truth = np.zeros((C, K, K, O))
    for r in range(K):
        for s2 in range(K):
            patch = xr[:, :, r:r + stride * Ho:stride, s2:s2 + stride * Wo:stride]
            truth[:, r, s2, :] = np.einsum("nchw,nohw->co", patch, dyr)
    mr, fr = oracle.errors(got.reshape(-1), truth.reshape(-1), float(np.sqrt(np.mean(truth ** 2))))
    assert mr <= 1e-3 and fr <= 1e-4, (mr, fr)


def test_conv_backward_weights_rejects_what_the_kernels_do_not_take(nz):
    import torch
    x, dy = torch.zeros((1, 1, 40, 40), device="cuda"), torch.zeros((1, 1, 29, 29), device="cuda")
    with pytest.raises(nz.NzHipError) as e:                      # 12 x 12 = 144 taps
        nz.conv2d_backward_weights(torch.zeros((1, 1, 144, 1), device="cuda"), x, dy, 12, 12, 1, 0)
    assert e.value.status == -3


def test_conv1x1_backward_weights_float_tolerance(nz, oracle):
    N, C, H, W, O = 3, 96, 20, 28, 80
    rng = np.random.default_rng(19)
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    dy = rng.standard_normal((N, O, H, W)).astype(np.float32)
    dw0 = rng.standard_normal((1, 1, C, O)).astype(np.float32)
    got = host(nz.conv2d_backward_weights(dev(dw0), dev(x), dev(dy), 1, 1, 1, 0))
    xr, dyr = oracle.round_f16(x).astype(np.float64), oracle.round_f16(dy).astype(np.float64)
    truth = dw0.astype(np.float64) + np.einsum("nchw,nohw->co", xr, dyr).reshape(1, 1, C, O)
    mr, fr = oracle.errors(got, truth, float(np.sqrt(np.mean(truth ** 2))))
    assert mr <= 1e-3 and fr <= 1e-4, (mr, fr)


def test_conv2d_backward_weights_float_tolerance(nz, oracle):
    N, C, H, W, O = 2, 48, 20, 72, 80
    rng = np.random.default_rng(9)
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    dy = rng.standard_normal((N, O, H, W)).astype(np.float32)
    got = host(nz.conv2d_backward_weights(dev(np.zeros((1, 1, C * 9, O))), dev(x), dev(dy), 3, 3, 1, 1))
    xr, dyr = oracle.round_f16(x).astype(np.float64), oracle.round_f16(dy).astype(np.float64)
    xp = np.pad(xr, ((0, 0), (0, 0), (1, 1), (1, 1)))
    truth = np.zeros((C, 3, 3, O))
    for r in range(3):
        for sx in range(3):
            truth[:, r, sx, :] = np.einsum("nchw,nohw->co", xp[:, :, r:r + H, sx:sx + W], dyr)
    truth = truth.reshape(1, 1, C * 9, O)
    mr, fr = oracle.errors(got, truth, float(np.sqrt(np.mean(truth ** 2))))
    assert mr <= 1e-3 and fr <= 1e-4, (mr, fr)


def test_conv2d_backward_weights_few_channels_float_tolerance(nz, oracle):
    # the streaming kernel on float data against an fp64 sum of the rounded operands
    N, C, H, W, O = 3, 3, 50, 300, 1
    rng = np.random.default_rng(10)
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    dy = rng.standard_normal((N, O, H, W)).astype(np.float32)
    got = host(nz.conv2d_backward_weights(dev(np.zeros((N, 1, C * 9, O))), dev(x), dev(dy), 3, 3, 1, 1))
    xr, dyr = oracle.round_f16(x).astype(np.float64), oracle.round_f16(dy).astype(np.float64)
    xp = np.pad(xr, ((0, 0), (0, 0), (1, 1), (1, 1)))
    truth = np.zeros((N, C, 3, 3, O))
    for r in range(3):
        for sx in range(3):
            truth[:, :, r, sx, :] = np.einsum("nchw,nohw->nco", xp[:, :, r:r + H, sx:sx + W], dyr)
    truth = truth.reshape(N, 1, C * 9, O)
    mr, fr = oracle.errors(got, truth, float(np.sqrt(np.mean(truth ** 2))))
    assert mr <= 1e-3 and fr <= 1e-4, (mr, fr)


@pytest.mark.parametrize("N,O,H,W", [(1, 1, 1, 1), (3, 5, 7, 9), (2, 40, 9, 30), (4, 128, 16, 24), (5, 1, 30, 70), (2, 33, 1, 130), (3, 50, 6, 10), (7, 17, 8, 36)])
def test_conv2d_backward_bias_equals_the_two_step_chain_bit_for_bit(nz, oracle, N, O, H, W):
    """One kernel for Col2Img.backward (transpose) + Add.backward (sum over the batch onto the gradient already
    there): the same additions in the same order, so float data agree bit for bit with the oracle's chain."""
    rng = np.random.default_rng(N + 3 * O + 5 * H + 7 * W)
    dz = rng.standard_normal((N, O, H, W)).astype(np.float32)
    base = rng.standard_normal((1, 1, H * W, O)).astype(np.float32)
    # with a batch of one the reference's Add.backward copies instead of adding (equal shapes); the kernel always adds
    want = oracle.add_backward(base, oracle.col2im_backward(dz)) if N > 1 else base + oracle.col2im_backward(dz)
    got = host(nz.conv2d_backward_bias(dev(base), dev(dz)))
    assert np.array_equal(got, want)


@pytest.mark.parametrize("N,O,H,W", [(3, 5, 7, 9), (2, 40, 9, 30), (4, 128, 16, 24), (2, 33, 1, 130)])
def test_conv2d_backward_relu_bias_equals_relu_backward_then_bias(nz, oracle, N, O, H, W):
    rng = np.random.default_rng(2 * N + 3 * O + 5 * H + 7 * W)
    y = np.maximum(rng.standard_normal((N, O, H, W)), 0).astype(np.float32)       # a ReLU output: zeros and positives
    dy = rng.standard_normal((N, O, H, W)).astype(np.float32)
    base = rng.standard_normal((1, 1, H * W, O)).astype(np.float32)
    dz_want = oracle.relu_backward(y, dy)
    db_want = oracle.add_backward(base, oracle.col2im_backward(dz_want))
    db = dev(base)
    dz = nz.conv2d_backward_relu_bias(db, dev(y), dev(dy))
    assert np.array_equal(host(dz), dz_want) and np.array_equal(host(db), db_want)


def test_conv2d_backward_weights_rejects_what_it_does_not_cover(nz):
    from neuzephyr_amd.capi import NzHipError
    with pytest.raises(NzHipError) as e:      # stride 5
        nz.conv2d_backward_weights(dev(np.zeros((1, 1, 18, 3))), dev(np.zeros((1, 2, 11, 11))), dev(np.zeros((1, 3, 3, 3))), 3, 3, 5, 1)
    assert e.value.status == -3
    with pytest.raises(NzHipError) as e:      # a kernel larger than the padded input
        nz.conv2d_backward_weights(dev(np.zeros((1, 1, 50, 3))), dev(np.zeros((1, 2, 2, 2))), dev(np.zeros((1, 3, 1, 1))), 5, 5, 1, 0)
    assert e.value.status == -2


def _random_conv_geometries(count, seed, many_images=False):
    """Seeded geometries across every conv route: few and many channels, 1x1 to 7x7 kernels (also rectangular),
    strides 1..4, paddings up to the kernel's reach and one beyond, shared and per-sample weights. many_images: enough
    images that the implicit-GEMM kernels have a workgroup for every compute unit (instead of the few-patch routes)."""
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        N = int(rng.integers(24, 97)) if many_images else int(rng.integers(1, 7))
        C = int(rng.choice([1, 2, 3, 5, 8, 16, 24, 40, 70, 130, 200]))
        O = int(rng.choice([1, 2, 3, 5, 17, 64, 70, 130]))
        Kh, Kw = int(rng.integers(1, 8)), int(rng.integers(1, 8))
        if rng.random() < 0.6:
            Kw = Kh
        stride = int(rng.choice([1, 1, 1, 2, 2, 3, 4]))
        pad = int(rng.integers(0, max(Kh, Kw) + 1))
        H, W = int(rng.integers(Kh, 41)), int(rng.choice([8, 12, 16, 20, 28, 30, 33, 40, 64, 70]))
        if W + 2 * pad < Kw or H + 2 * pad < Kh or C * Kh * Kw * O > 300000 or N * C * H * W > 6000000 or N * O * H * W > 12000000:
            continue
        wb = N if rng.random() < 0.25 else 1
        cases.append((N, C, H, W, O, Kh, Kw, stride, pad, wb))
    return cases


@pytest.mark.parametrize("N,C,H,W,O,Kh,Kw,stride,pad,wb", _random_conv_geometries(48, 2024) + _random_conv_geometries(32, 7, many_images=True))
def test_random_conv_geometries_forward_and_gradients_bit_exact(nz, oracle, N, C, H, W, O, Kh, Kw, stride, pad, wb):
    """Forward, weight gradient and (where the entry point covers the geometry) data gradient of one seeded random layer
    on integer-valued data against the oracle; whatever route the shape takes, the sums are exact."""
    from neuzephyr_amd.capi import NzHipError
    rng = np.random.default_rng(N + 3 * C + 5 * H + 7 * W + 11 * O + 13 * Kh + 17 * Kw + 19 * stride + 23 * pad)
    Ho, Wo = (H + 2 * pad - Kh) // stride + 1, (W + 2 * pad - Kw) // stride + 1
    x = rng.integers(-3, 4, size=(N, C, H, W)).astype(np.float32)
    ws = [rng.integers(-2, 3, size=(O, C, Kh, Kw)).astype(np.float32) for _ in range(wb)]
    w_ref = np.concatenate([oracle.weights_oihw_to_ref(w) for w in ws], axis=0)
    bias = rng.integers(-2, 3, size=(O,)).astype(np.float32)
    got = host(nz.conv2d_forward(dev(x), dev(w_ref), dev(bias), Kh, Kw, stride, pad, relu=True))
    for n in range(N):
        truth = np.maximum(oracle.conv2d_direct_f64(x[n:n + 1], ws[n if wb > 1 else 0], None, stride, pad) + bias.reshape(1, O, 1, 1), 0)
        assert np.array_equal(got[n:n + 1].astype(np.float64), truth), ("forward", n)
    dy = rng.integers(-3, 4, size=(N, O, Ho, Wo)).astype(np.float32)
    dw0 = rng.integers(-4, 5, size=w_ref.shape).astype(np.float32)
    want_dw = oracle.conv2d_backward_weights(dw0.copy(), x, dy, Kh, Kw, pad, stride)
    assert np.array_equal(host(nz.conv2d_backward_weights(dev(dw0), dev(x), dev(dy), Kh, Kw, stride, pad)), want_dw), "weights"
    dx0 = rng.integers(-3, 4, size=x.shape).astype(np.float32)
    if Kh == Kw and pad <= Kh - 1:
        for accumulate in (True, False):
            want_dx = oracle.conv2d_backward_data(dx0.copy() if accumulate else np.zeros_like(dx0), dy, w_ref, Kh, Kw, pad, stride)
            got_dx = host(nz.conv2d_backward_data(dev(dx0), dev(dy), dev(w_ref), Kh, Kw, stride, pad, accumulate=accumulate))
            assert np.array_equal(got_dx, want_dx), ("data", accumulate)
    else:
        with pytest.raises(NzHipError):
            nz.conv2d_backward_data(dev(dx0), dev(dy), dev(w_ref), Kh, Kw, stride, pad)
