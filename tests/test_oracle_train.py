"""Pins the oracle's optimizer steps: SGD against its closed form, Adam against the host formula the
reference's own test uses (test/Test.cpp:2398-2452) and against invariants of the update."""
import numpy as np


def test_sgd_closed_form(oracle):
    rng = np.random.default_rng(1)
    data = rng.uniform(-10, 10, 72).astype(np.float32)
    grad = rng.uniform(-10, 10, 72).astype(np.float32)
    lr = np.float32(0.01)
    assert np.array_equal(oracle.sgd_step(data, grad, float(lr)), data - lr * grad)   # test/Test.cpp:2230-2265


def test_adam_two_steps_match_the_reference_test_formula(oracle):
    rng = np.random.default_rng(2)
    n = 72
    data = rng.uniform(-10, 10, n).astype(np.float32)
    grad = rng.uniform(-10, 10, n).astype(np.float32)
    lr, b1, b2, eps = np.float32(0.01), np.float32(0.9), np.float32(0.999), np.float32(1e-6)
    m = np.zeros(n, np.float32); v = np.zeros(n, np.float32)
    want = data.copy()
    for it in (1, 2):                                             # test/Test.cpp:2426-2441, in double
        m = b1 * m + (1 - b1) * grad
        v = b2 * v + (1 - b2) * grad * grad
        mm = m.astype(np.float64) / (1 - float(b1) ** it)
        vv = v.astype(np.float64) / (1 - float(b2) ** it)
        want = want - (float(lr) / (np.sqrt(vv) + float(eps))) * mm
    d, m_o, v_o = data, np.zeros(n, np.float32), np.zeros(n, np.float32)
    for it in (1, 2):
        d, m_o, v_o = oracle.adam_step(d, m_o, v_o, grad, float(lr), float(b1), float(b2), float(eps), it)
    assert np.allclose(d, want, rtol=1e-5, atol=1e-6)            # the tolerance of the reference's EXPECT_EQ
    assert np.allclose(m_o, m, rtol=1e-6) and np.allclose(v_o, v, rtol=1e-6)


def test_adam_first_step_moves_by_lr_against_the_gradient_sign(oracle):
    # t = 1: m_hat = g, v_hat = g*g  ->  step = lr * g / (|g| + eps)
    grad = np.array([3.0, -0.5, 1e-3, -20.0], np.float32)
    data = np.zeros(4, np.float32)
    d, m, v = oracle.adam_step(data, np.zeros(4, np.float32), np.zeros(4, np.float32), grad, 0.25, 0.9, 0.999, 1e-8, 1)
    assert np.allclose(d, -0.25 * np.sign(grad), rtol=1e-4)
    # 1 - 0.999f is 0.00099998713 in fp32 (the kernel computes it in fp32 too): 1.3e-5 off 0.001
    assert np.allclose(m, 0.1 * grad, rtol=1e-6) and np.allclose(v, 0.001 * grad * grad, rtol=1e-4)
    # a zero gradient leaves the parameter alone
    d0, _, _ = oracle.adam_step(np.ones(3, np.float32), np.zeros(3, np.float32), np.zeros(3, np.float32),
                                np.zeros(3, np.float32), 0.1, 0.9, 0.999, 1e-6, 1)
    assert np.array_equal(d0, np.ones(3, np.float32))


def test_softmax_and_jacobian_loop_nests(oracle):
    # test/Test.cpp:1823-1832 (softmax) and :1782-1795 (Jacobian), plus what the mathematics fixes
    rng = np.random.default_rng(4)
    x = rng.uniform(-10, 10, (2, 3, 12, 1)).astype(np.float32)
    want = np.empty_like(x)
    for i in range(2):
        for j in range(3):
            e = np.exp(x[i, j, :, 0].astype(np.float64))
            want[i, j, :, 0] = (e / e.sum()).astype(np.float32)
    s = oracle.softmax(x)
    assert np.allclose(s, want, rtol=1e-6, atol=1e-9)
    assert np.allclose(s.sum(axis=2), 1.0, atol=1e-6)
    assert np.allclose(oracle.softmax(x + 3.0), s, rtol=1e-5)          # shift invariance
    J = oracle.softmax_jacobian(s)
    for i in range(2):
        for j in range(3):
            v = s[i, j, :, 0]
            assert np.array_equal(J[i, j], (np.diag(v * (1 - v)) - np.outer(v, v) * (1 - np.eye(12, dtype=np.float32))).astype(np.float32))
    assert np.allclose(J.sum(axis=3), 0.0, atol=1e-6)                   # rows of a softmax Jacobian sum to zero
    assert np.array_equal(J, J.transpose(0, 1, 3, 2))                   # and it is symmetric
    # row-vector input: same Jacobian, gradient multiplied from the left
    dy = rng.uniform(-1, 1, (2, 3, 12, 1)).astype(np.float32)
    col = oracle.softmax_backward(s, dy)
    row = oracle.softmax_backward(s.reshape(2, 3, 1, 12), dy.reshape(2, 3, 1, 12))
    assert np.allclose(col.reshape(-1), row.reshape(-1), rtol=1e-6, atol=1e-7)
    # closed form s * (dy - <s, dy>) within the fp16 rounding of the GEMM operands
    ref = s * (dy - (s * dy).sum(axis=2, keepdims=True))
    assert np.allclose(col, ref, atol=2e-3)
