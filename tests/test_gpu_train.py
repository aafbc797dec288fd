"""fp32-exact matmul (Tensor::operator*) and optimizer steps on the GPU against the CPU oracle,
through the C-ABI. The matmul accumulates with FMAs in ascending k exactly like the oracle's scalar
loop: results are compared bit for bit, also on float data."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


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


def test_matmul_f32_reference_literal_vector(nz):
    # test/Test.cpp:119-184
    A = np.arange(1, 13, dtype=np.float32).reshape(2, 1, 2, 3)
    B = np.arange(1, 19, dtype=np.float32).reshape(1, 3, 3, 2)
    want = np.array([22, 28, 49, 64, 58, 64, 139, 154, 94, 100, 229, 244, 76, 100, 103, 136, 220, 244, 301, 334, 364, 388,
                     499, 532], np.float32).reshape(2, 3, 2, 2)
    assert np.array_equal(host(nz.matmul_f32(dev(A), dev(B))), want)


@pytest.mark.parametrize("sa,sb", [((1, 1, 1, 1), (1, 1, 1, 1)), ((2, 3, 5, 7), (2, 3, 7, 6)), ((2, 1, 33, 17), (1, 3, 17, 130)),
                                   ((1, 1, 129, 65), (1, 1, 65, 131)), ((1, 1, 300, 40), (1, 1, 40, 260)),
                                   ((3, 2, 64, 16), (1, 1, 16, 64)), ((1, 1, 7, 1000), (1, 1, 1000, 5))])
def test_matmul_f32_bit_identical_to_the_oracle(nz, oracle, sa, sb):
    rng = np.random.default_rng(sum(sa) * 7 + sum(sb))
    A = rng.standard_normal(sa).astype(np.float32)
    B = rng.standard_normal(sb).astype(np.float32)
    # 1 + 2^-12 is not a half: a kernel that rounded its operands to fp16 would lose it
    A.reshape(-1)[0] = 1 + 2.0 ** -12
    got = host(nz.matmul_f32(dev(A), dev(B)))
    assert np.array_equal(got, oracle.general_matmul(A, B))


def test_matmul_f32_is_one_fma_chain_in_ascending_k(nz, oracle):
    # operands spread over 20 binades: a different order of the additions, or products rounded before they are added,
    # would change most outputs (the kernel's fp32 MFMAs must behave like the scalar chain)
    rng = np.random.default_rng(99)
    A = (rng.standard_normal((1, 1, 160, 777)) * np.exp2(rng.integers(-10, 11, size=(1, 1, 160, 777)))).astype(np.float32)
    B = (rng.standard_normal((1, 1, 777, 200)) * np.exp2(rng.integers(-10, 11, size=(1, 1, 777, 200)))).astype(np.float32)
    got = host(nz.matmul_f32(dev(A), dev(B)))
    want = oracle.general_matmul(A, B)
    assert np.array_equal(got, want)
    # and the chain is not what numpy's pairwise float32 product gives: the check above can tell orders apart
    assert not np.array_equal(want[0, 0], A[0, 0] @ B[0, 0])


def test_matmul_f32_rejects_bad_shapes(nz):
    with pytest.raises(nz.NzHipError):
        nz.matmul_f32(dev(np.zeros((1, 1, 2, 3))), dev(np.zeros((1, 1, 4, 2))))
    with pytest.raises(nz.NzHipError):
        nz.matmul_f32(dev(np.zeros((2, 1, 2, 3))), dev(np.zeros((3, 1, 3, 2))))


def test_sgd_step_bit_exact(nz, oracle):
    rng = np.random.default_rng(41)
    for n in (1, 72, 4097):
        data = rng.uniform(-10, 10, n).astype(np.float32)
        grad = rng.uniform(-10, 10, n).astype(np.float32)
        got = host(nz.sgd_step(dev(data), dev(grad), 0.01))
        assert np.allclose(got, oracle.sgd_step(data, grad, 0.01), rtol=0, atol=0) or \
            np.max(np.abs(got - oracle.sgd_step(data, grad, 0.01))) <= np.spacing(np.float32(10.0))   # mul+sub may fuse


def test_adam_steps_match_oracle(nz, oracle):
    rng = np.random.default_rng(43)
    n = 4099
    data = rng.uniform(-10, 10, n).astype(np.float32)
    grad = rng.uniform(-10, 10, n).astype(np.float32)
    d, m, v = dev(data), dev(np.zeros(n)), dev(np.zeros(n))
    do, mo, vo = data, np.zeros(n, np.float32), np.zeros(n, np.float32)
    for t in (1, 2, 3):
        nz.adam_step(d, m, v, dev(grad), 0.01, 0.9, 0.999, 1e-6, t)
        do, mo, vo = oracle.adam_step(do, mo, vo, grad, 0.01, 0.9, 0.999, 1e-6, t)
    assert np.allclose(host(d), do, rtol=1e-5, atol=1e-6)        # the reference's own comparison tolerance
    assert np.allclose(host(m), mo, rtol=1e-6, atol=1e-7) and np.allclose(host(v), vo, rtol=1e-6, atol=1e-7)
    with pytest.raises(nz.NzHipError):
        nz.adam_step(d, m, v, dev(grad), 0.01, 0.9, 0.999, 1e-6, 0)


def test_many_tensor_steps_equal_the_one_tensor_calls(nz):
    """One launch for up to 16 tensors: every element gets the arithmetic of the one-tensor call (bit-identical),
    for sizes with and without 16-byte tails, an unaligned tensor, an empty one, and more tensors than one launch takes."""
    import torch
    rng = np.random.default_rng(59)
    sizes = [1, 3, 4, 27, 72, 1024, 4097, 0, 260100, 16, 5, 300000, 7, 64, 129, 2, 33, 1000, 6]      # 19 tensors: two launches
    def tensors(seed, offset_one=True):
        r = np.random.default_rng(seed)
        out = []
        for i, n in enumerate(sizes):
            base = dev(r.uniform(-10, 10, n + 1).astype(np.float32))
            out.append(base[1:] if (offset_one and i == 5) else base[:n])       # tensor 5 is not 16-byte aligned
        return out
    # fill
    a, b = tensors(1), tensors(1)
    nz.fill_many(a, 0.25)
    for t in b: nz.fill(t, 0.25)
    assert all(torch.equal(x, y) for x, y in zip(a, b))
    # SGD
    a, b, g = tensors(2), tensors(2), tensors(3)
    nz.sgd_step_many(a, g, 0.01)
    for x, gg in zip(b, g):
        if x.numel(): nz.sgd_step(x, gg, 0.01)
    assert all(torch.equal(x, y) for x, y in zip(a, b))
    # Adam, two updates with consecutive step counts per tensor as ComputeGraph::update produces them
    a, b, g = tensors(4), tensors(4), tensors(5)
    ma, mb = [torch.zeros_like(x) for x in a], [torch.zeros_like(x) for x in b]
    va, vb = [torch.zeros_like(x) for x in a], [torch.zeros_like(x) for x in b]
    count = 0
    for update in range(2):
        ts = list(range(count + 1, count + 1 + len(sizes)))
        count += len(sizes)
        nz.adam_step_many(a, ma, va, g, ts, 0.01, 0.9, 0.999, 1e-6)
        for x, m, v, gg, t in zip(b, mb, vb, g, ts):
            if x.numel(): nz.adam_step(x, m, v, gg, 0.01, 0.9, 0.999, 1e-6, t)
    assert all(torch.equal(x, y) for x, y in zip(a, b))
    assert all(torch.equal(x, y) for x, y in zip(ma, mb)) and all(torch.equal(x, y) for x, y in zip(va, vb))
    with pytest.raises(nz.NzHipError):
        nz.adam_step_many(a[:2], ma[:2], va[:2], g[:2], [1, 0], 0.01, 0.9, 0.999, 1e-6)


def test_softmax_forward_jacobian_backward(nz, oracle):
    rng = np.random.default_rng(47)
    for shape in [(2, 3, 12, 1), (1, 2, 1, 300), (3, 1, 1000, 1), (1, 1, 1, 1)]:
        x = rng.uniform(-10, 10, shape).astype(np.float32)
        s = host(nz.softmax(dev(x)))
        so = oracle.softmax(x)
        assert np.allclose(s, so, rtol=2e-6, atol=1e-9), shape          # fast exp + tree sum vs expf + serial sum
        J = host(nz.softmax_jacobian(dev(so)))
        assert np.array_equal(J, oracle.softmax_jacobian(so)), shape
        dy = rng.uniform(-10, 10, shape).astype(np.float32)
        want = oracle.softmax_backward(so, dy)
        got = host(nz.softmax_backward_gemm(dev(so), dev(dy)))      # Jacobian in memory, then the GEMM entry
        assert got.shape == want.shape and np.allclose(got, want, rtol=1e-5, atol=1e-6), shape
        # the fused kernel adds in ascending j like the oracle's GEMM: the same bits
        fused = host(nz.softmax_backward(dev(so), dev(dy)))
        assert fused.shape == want.shape and np.array_equal(fused, want), shape


def test_softmax_backward_fused_sizes(nz, oracle):
    """Chunk boundaries of the fused kernel (1024 entries per LDS chunk, 256 outputs per workgroup), fp16
    subnormal Jacobian entries (s_i s_j far below 6e-5) and the closed form dx = s * (dy - <s, dy>)."""
    rng = np.random.default_rng(48)
    for shape in [(1, 1, 255, 1), (2, 1, 1, 256), (1, 2, 1024, 1), (1, 1, 1, 1025), (2, 2, 2303, 1), (1, 1, 4097, 1)]:
        x = rng.uniform(-4, 4, shape).astype(np.float32)
        so = oracle.softmax(x)
        dy = rng.uniform(-3, 3, shape).astype(np.float32)
        want = oracle.softmax_backward(so, dy)
        got = host(nz.softmax_backward(dev(so), dev(dy)))
        assert np.array_equal(got, want), shape
        s64, g64 = so.astype(np.float64), dy.astype(np.float64)
        axis = 2 if shape[2] > 1 else 3
        closed = s64 * (g64 - (s64 * g64).sum(axis=axis, keepdims=True))
        assert np.abs(got - closed).max() <= 2e-3 * np.abs(closed).max(), shape   # fp16 operands
    # a gradient beyond fp16 range rounds to infinity in the GEMM operands, and so it does here
    so = oracle.softmax(np.zeros((1, 1, 8, 1), np.float32))
    dy = np.full((1, 1, 8, 1), 1e5, np.float32)
    got = host(nz.softmax_backward(dev(so), dev(dy)))
    want = oracle.softmax_backward(so, dy)
    assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(got[~np.isnan(got)], want[~np.isnan(want)])


def test_optimizer_steps_vector_and_tail_paths(nz, oracle):
    """Four elements per thread on 16-byte aligned arrays plus the n % 4 tail, and one element per thread on a
    view that is only 4-byte aligned: the same bits per element, and the oracle's values at the tolerance of
    the tests above."""
    rng = np.random.default_rng(49)
    for n in (1, 3, 4, 1023, 1024, 1027, 262147):
        base = [rng.standard_normal(n + 1).astype(np.float32) for _ in range(2)]
        base.append((0.1 * rng.standard_normal(n + 1)).astype(np.float32))
        base.append(np.abs(0.1 * rng.standard_normal(n + 1)).astype(np.float32))
        vals = [np.ascontiguousarray(a[1:]) for a in base]            # data, grad, m, v
        results = []
        for unaligned in (False, True):
            d, g, m, v = (dev(a)[1:] for a in base) if unaligned else (dev(a) for a in vals)
            assert (d.data_ptr() % 16 != 0) == unaligned
            d_sgd = d.clone() if not unaligned else dev(base[0])[1:]
            nz.sgd_step(d_sgd, g, 0.05)
            nz.adam_step(d, m, v, g, 0.01, 0.9, 0.999, 1e-6, 3)
            results.append([host(t) for t in (d_sgd, d, m, v)])
        for a, b in zip(*results):
            assert np.array_equal(a, b), n
        sgd, d, m, v = results[0]
        assert np.max(np.abs(sgd - oracle.sgd_step(vals[0], vals[1], 0.05))) <= np.spacing(np.float32(8.0)), n
        do, mo, vo = oracle.adam_step(vals[0], vals[2], vals[3], vals[1], 0.01, 0.9, 0.999, 1e-6, 3)
        assert np.allclose(d, do, rtol=1e-5, atol=1e-6), n
        assert np.allclose(m, mo, rtol=1e-6, atol=1e-7) and np.allclose(v, vo, rtol=1e-6, atol=1e-7), n
