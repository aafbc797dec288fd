"""Pins the oracle's im2col / col2im / bias / ReLU / Conv2d graph
(src/OperationKernels.cu:1308-1328, :1364-1376, :12-24, :230-235 and
src/Model.cu:244-263 of the reference) against the layout specification the
reference's own tests hold as loop nests (test/Test.cpp:2903-2935, :3090-3099)
and against an independent direct convolution."""
import numpy as np
import pytest


def _spec_im2col(x, k_h, k_w, stride, pad):
    """The loop nest of TensorBasic.img2colTest (test/Test.cpp:2903-2935)."""
    n, c, h, w = x.shape
    H_out = (h + 2 * pad - k_h) // stride + 1
    W_out = (w + 2 * pad - k_w) // stride + 1
    flat = x.reshape(-1)
    out = np.zeros(n * H_out * W_out * k_h * k_w * c, np.float32)
    for b in range(n):
        for i in range(H_out):
            for j in range(W_out):
                h_start, w_start = i * stride - pad, j * stride - pad
                for r in range(k_h):
                    h_in = h_start + r
                    for s in range(k_w):
                        w_in = w_start + s
                        for c_in in range(c):
                            val = 0.0
                            if 0 <= h_in < h and 0 <= w_in < w:
                                val = flat[b * (c * h * w) + c_in * (h * w) + h_in * w + w_in]
                            out[b * (H_out * W_out * k_h * k_w * c) + (i * W_out + j) * (k_h * k_w * c)
                                + c_in * (k_h * k_w) + r * k_w + s] = val
    return out.reshape(n, 1, H_out * W_out, k_h * k_w * c)


@pytest.mark.parametrize("shape,k_h,k_w,stride,pad", [
    ((2, 3, 4, 5), 3, 3, 1, 1),      # the reference test's own case
    ((1, 1, 1, 1), 1, 1, 1, 0),
    ((2, 2, 7, 6), 3, 2, 2, 0),      # non-square kernel, stride 2, no padding
    ((1, 3, 8, 9), 2, 4, 2, 2),      # padding 2
    ((3, 1, 5, 5), 5, 5, 1, 2),      # kernel as large as the image
    ((2, 4, 6, 6), 1, 1, 3, 0),
])
def test_im2col_matches_reference_spec(oracle, shape, k_h, k_w, stride, pad):
    x = np.random.default_rng(sum(shape)).uniform(0.1, 0.9, size=shape).astype(np.float32)
    assert np.array_equal(oracle.im2col(x, k_h, k_w, stride, pad), _spec_im2col(x, k_h, k_w, stride, pad))


def test_col2im_matches_reference_spec(oracle):
    # test/Test.cpp:3090-3099: expected[b][j][k][l] = in[b][(k*w + l)*c + j]
    n, c, h, w = 2, 3, 4, 5
    col = np.random.default_rng(3).uniform(0.1, 0.9, size=(n, 1, h * w, c)).astype(np.float32)
    expect = col.reshape(n, h, w, c).transpose(0, 3, 1, 2)
    assert np.array_equal(oracle.col2im(col, h, w), expect)
    assert not np.array_equal(oracle.col2im(col, h, w).reshape(n, 1, h * w, c), col)


def test_matrix_add_broadcast_and_relu_special_values(oracle):
    a = np.arange(2 * 3 * 2 * 2, dtype=np.float32).reshape(2, 3, 2, 2)
    b = np.array([10, 20, 30, 40], np.float32).reshape(1, 1, 2, 2)
    assert np.array_equal(oracle.matrix_add(a, b), a + b)
    b2 = np.arange(12, dtype=np.float32).reshape(1, 3, 2, 2) * 100
    assert np.array_equal(oracle.matrix_add(a, b2), a + b2)
    assert np.array_equal(oracle.matrix_add(b2, a), a + b2)
    v = np.array([np.nan, -0.0, 0.0, -1.5, 2.5, np.inf, -np.inf, 1e-45], np.float32)
    r = oracle.relu(v)
    assert np.array_equal(r, np.array([0, 0, 0, 0, 2.5, np.inf, 0, 1e-45], np.float32))
    assert not np.signbit(r[1])                                # -0 -> +0, NaN -> 0 (x > 0 ? x : 0)


@pytest.mark.parametrize("N,C,H,W,O,k_h,k_w,stride,pad,w_batch", [
    (2, 3, 6, 7, 4, 3, 3, 1, 1, 1),
    (2, 3, 6, 7, 4, 3, 3, 1, 1, 2),     # Model::Conv2d allocates one weight copy per sample
    (1, 2, 9, 8, 3, 2, 3, 2, 0, 1),
    (3, 1, 5, 5, 1, 3, 3, 1, 2, 1),
])
def test_conv_graph_equals_direct_convolution_on_integers(oracle, N, C, H, W, O, k_h, k_w, stride, pad, w_batch):
    rng = np.random.default_rng(N + C + H + W + O)
    x = rng.integers(-4, 5, size=(N, C, H, W)).astype(np.float32)
    w = rng.integers(-3, 4, size=(O, C, k_h, k_w)).astype(np.float32)
    bias = rng.integers(-2, 3, size=(O,)).astype(np.float32)
    Ho, Wo = oracle.out_hw(H, W, k_h, k_w, stride, pad)
    w_ref = oracle.weights_oihw_to_ref(w)
    if w_batch > 1:
        w_ref = np.ascontiguousarray(np.broadcast_to(w_ref, (w_batch,) + w_ref.shape[1:]))
    y = oracle.conv2d_graph(x, w_ref, oracle.bias_channel_to_ref(bias, Ho * Wo), k_h, k_w, stride, pad, relu=True)
    truth = oracle.conv2d_direct_f64(x, w, bias, stride, pad, relu=True)
    assert np.array_equal(y.astype(np.float64), truth)          # small integers: exact in both


def test_conv_graph_per_pixel_bias_and_tolerance(oracle):
    # the reference's bias parameter is [1,1,Ho*Wo,O]: a different value per pixel and channel
    N, C, H, W, O = 2, 5, 10, 9, 6
    x = oracle.fill((N, C, H, W), 61, "normal", 0.0, 1.0)
    w = oracle.fill((O, C, 3, 3), 62, "normal", 0.0, 0.2)
    Ho, Wo = oracle.out_hw(H, W, 3, 3, 1, 1)
    bias_px = oracle.fill((1, 1, Ho * Wo, O), 63, "uniform", -0.5, 0.5)
    y = oracle.conv2d_graph(x, oracle.weights_oihw_to_ref(w), bias_px, 3, 3, 1, 1, relu=False)
    truth = oracle.conv2d_direct_f64(x, w, None, 1, 1, relu=False)
    truth = truth + bias_px.reshape(Ho, Wo, O).transpose(2, 0, 1)[None].astype(np.float64)
    mr, fr = oracle.errors(y, truth, float(np.sqrt(np.mean(truth ** 2))))
    assert mr <= 1e-5 and fr <= 1e-6
