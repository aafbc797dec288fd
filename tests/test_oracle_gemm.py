"""Pins the oracle's GEMM (src/OperationKernels.cu:821-844 + :914-1026 of the
reference) without retyping its formula: the reference's own literal vectors,
integer exactness against int64 arithmetic, structured matrices with known
answers, an explicit k-ascending fp32 summation written with numpy scalars,
and the fp64 truth with the classical error bound."""
import json
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(__file__), "golden", "matmul_broadcast.json")


def _gold():
    with open(GOLD) as f:
        g = json.load(f)
    A = np.array(g["A"], np.float32).reshape(g["shapeA"])
    B = np.array(g["B"], np.float32).reshape(g["shapeB"])
    C = np.array(g["C"], np.float32).reshape(g["shapeC"])
    return A, B, C


def test_reference_literal_vectors(oracle):
    A, B, C = _gold()
    assert np.array_equal(oracle.tensorcore_gemm(A, B), C)
    # TensorCore.TensorCoreGEMMTest asserts fp16 path == fp32 path on these inputs
    assert np.array_equal(oracle.general_matmul(A, B), C)


@pytest.mark.parametrize("M,K,N", [(1, 1, 1), (3, 5, 2), (16, 16, 16), (17, 33, 15), (64, 100, 130), (130, 257, 67)])
@pytest.mark.parametrize("trans_b", [False, True])
def test_integer_inputs_are_exact(oracle, M, K, N, trans_b):
    rng = np.random.default_rng(M * 1000 + K * 10 + N)
    A = rng.integers(-8, 9, size=(M, K)).astype(np.float32)
    B = rng.integers(-8, 9, size=(K, N)).astype(np.float32)
    expect = (A.astype(np.int64) @ B.astype(np.int64)).astype(np.float32)  # |sums| < 2^24: exact in any order
    Bop = np.ascontiguousarray(B.T) if trans_b else B
    assert np.array_equal(oracle.gemm(A, Bop, trans_b=trans_b), expect)


def test_identity_permutation_and_ones(oracle):
    n = 70
    X = oracle.fill((n, n), 11, "uniform", -4.0, 4.0)
    Xr = oracle.round_f16(X)
    eye = np.eye(n, dtype=np.float32)
    assert np.array_equal(oracle.gemm(eye, X), Xr)          # I*X = f16(X)
    assert np.array_equal(oracle.gemm(X, eye), Xr)
    perm = np.random.default_rng(0).permutation(n)
    P = eye[perm]
    assert np.array_equal(oracle.gemm(P, X), Xr[perm])       # row permutation
    # a transposed operand would fail here unless X is symmetric
    assert not np.array_equal(oracle.gemm(eye, X), Xr.T)
    ones = np.ones((1, n), np.float32)
    ints = np.random.default_rng(1).integers(-100, 100, size=(n, 9)).astype(np.float32)
    assert np.array_equal(oracle.gemm(ones, ints)[0], ints.sum(axis=0))


def test_k_ascending_fp32_accumulation_bitwise(oracle):
    A = oracle.fill((6, 300), 21, "normal", 0.0, 1.0)
    B = oracle.fill((300, 5), 22, "normal", 0.0, 1.0)
    Ar = A.astype(np.float16).astype(np.float32)             # numpy's converter, not the oracle's
    Br = B.astype(np.float16).astype(np.float32)
    expect = np.zeros((6, 5), np.float32)
    for i in range(6):
        for j in range(5):
            acc = np.float32(0)
            for k in range(300):
                acc = np.float32(acc + np.float32(Ar[i, k] * Br[k, j]))
            expect[i, j] = acc
    got = oracle.gemm(A, B)
    assert np.array_equal(got.view(np.uint32), expect.view(np.uint32))
    # blocked kernel boundaries (k > 256, n > 64, ragged rows) keep the same order
    A = oracle.fill((9, 777), 23, "uniform", -1.0, 1.0)
    B = oracle.fill((777, 131), 24, "uniform", -1.0, 1.0)
    Ar = A.astype(np.float16).astype(np.float32)
    Br = B.astype(np.float16).astype(np.float32)
    acc = np.zeros((9, 131), np.float32)
    for k in range(777):
        acc = (acc + Ar[:, k:k + 1] * Br[k:k + 1, :]).astype(np.float32)
    assert np.array_equal(oracle.gemm(A, B), acc)
    assert np.array_equal(oracle.gemm(A, np.ascontiguousarray(B.T), trans_b=True), acc)


def test_fp64_truth_and_error_bound(oracle):
    M, K, N = 96, 1000, 80
    A = oracle.fill((M, K), 31, "uniform", -1.0, 1.0)
    B = oracle.fill((K, N), 32, "uniform", -1.0, 1.0)
    Ar = A.astype(np.float16).astype(np.float64)
    Br = B.astype(np.float16).astype(np.float64)
    truth = Ar @ Br
    c64 = oracle.gemm_f64(A, B)
    assert np.max(np.abs(c64 - truth)) <= 1e-11
    c32 = oracle.gemm(A, B).astype(np.float64)
    bound = K * 2.0 ** -24 * (np.abs(Ar) @ np.abs(Br))       # Higham: |fl(sum)-sum| <= (K-1)u sum|a_i b_i|
    assert np.all(np.abs(c32 - truth) <= bound)
    max_rel, frob = oracle.errors(c32.astype(np.float32), truth, float(np.sqrt(np.mean(truth ** 2))))
    assert max_rel <= 1e-3 and frob <= 1e-4
    # unrounded operands differ: the rounding is really applied
    assert np.max(np.abs(truth - A.astype(np.float64) @ B.astype(np.float64))) > 1e-4


def test_rows_sampling_agrees_with_full(oracle):
    A = oracle.fill((40, 129), 41, "normal", 0.0, 1.0)
    B = oracle.fill((129, 70), 42, "normal", 0.0, 1.0)
    full32, full64 = oracle.gemm(A, B), oracle.gemm_f64(A, B)
    r32, r64 = oracle.gemm_rows(A, B, 7, 9)
    assert np.array_equal(r32, full32[7:16]) and np.array_equal(r64, full64[7:16])


@pytest.mark.parametrize("sa,sb", [((2, 1, 2, 3), (1, 3, 3, 2)), ((3, 2, 5, 7), (3, 2, 7, 4)),
                                    ((1, 1, 9, 6), (4, 1, 6, 1)), ((2, 3, 4, 5), (1, 1, 5, 6)),
                                    ((1, 3, 4, 5), (2, 1, 5, 6))])
def test_batched_broadcast_semantics(oracle, sa, sb):
    rng = np.random.default_rng(sum(sa) + sum(sb))
    A = rng.integers(-5, 6, size=sa).astype(np.float32)
    B = rng.integers(-5, 6, size=sb).astype(np.float32)
    got = oracle.tensorcore_gemm(A, B)
    n, c = max(sa[0], sb[0]), max(sa[1], sb[1])
    assert got.shape == (n, c, sa[2], sb[3])
    for i in range(n):
        for j in range(c):
            a = A[i if sa[0] > 1 else 0, j if sa[1] > 1 else 0].astype(np.int64)
            b = B[i if sb[0] > 1 else 0, j if sb[1] > 1 else 0].astype(np.int64)
            assert np.array_equal(got[i, j], (a @ b).astype(np.float32))


def test_linear_graph_equals_per_sample_gemv(oracle):
    # Model::Linear (src/Model.cu:87-103): W[1,1,OUT,IN] x[N,1,IN,1] -> [N,1,OUT,1], + bias [1,1,OUT,1]
    Nb, IN, OUT = 5, 37, 11
    x = oracle.fill((Nb, IN), 51, "normal", 0.0, 1.0)
    W = oracle.fill((OUT, IN), 52, "uniform", -0.3, 0.3)
    bias = oracle.fill((OUT,), 53, "uniform", -0.03, 0.03)
    g = oracle.tensorcore_gemm(W.reshape(1, 1, OUT, IN), x.reshape(Nb, 1, IN, 1))
    g = oracle.matrix_add(g, bias.reshape(1, 1, OUT, 1))
    expect = oracle.relu(g).reshape(Nb, OUT)
    assert np.array_equal(oracle.linear_graph(x, W, bias, relu=True), expect)
    assert np.array_equal(oracle.linear_graph(x, W, None, relu=False),
                          oracle.gemm(x, W, trans_b=True))


def test_fill_is_deterministic_and_distributed(oracle):
    a = oracle.fill((100_003,), 9, "uniform", -1.0, 1.0)
    oracle.set_num_threads(1)
    b = oracle.fill((100_003,), 9, "uniform", -1.0, 1.0)
    oracle.set_num_threads(max(1, os.cpu_count() or 1))
    assert np.array_equal(a, b)                              # independent of the thread count
    assert not np.array_equal(a, oracle.fill((100_003,), 10, "uniform", -1.0, 1.0))
    assert a.min() >= -1.0 and a.max() <= 1.0
    assert abs(a.mean()) < 0.01 and abs(a.var() - 1.0 / 3.0) < 0.01
    g = oracle.fill((200_001,), 3, "normal", 2.0, 0.5)
    assert abs(g.mean() - 2.0) < 0.01 and abs(g.std() - 0.5) < 0.01
    assert abs(np.mean(((g - 2.0) / 0.5) ** 4) - 3.0) < 0.1  # kurtosis of a Gaussian
