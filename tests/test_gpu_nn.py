"""Average pooling, binary cross-entropy and expand / compress on the GPU against the CPU oracle, through
the C-ABI. Pooling, its gradient, the loss gradient and expand / compress are compared bit for bit (same
additions in the same order, correctly rounded divisions); the loss value uses the fast logarithm and a
tree sum and is compared at 1e-5 relative."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

POOL_CASES = [((2, 3, 4, 5), 2, 2, 0), ((1, 2, 9, 7), 3, 1, 1), ((2, 1, 10, 10), 5, 2, 0), ((1, 1, 6, 8), 4, 3, 2),
              ((1, 3, 5, 5), 5, 1, 2), ((2, 2, 7, 3), 1, 1, 0), ((1, 1, 8, 8), 3, 2, 1), ((3, 5, 33, 47), 3, 2, 1),
              ((1, 1, 70, 300), 5, 2, 0), ((2, 2, 16, 16), 2, 2, 0), ((1, 1, 9, 9), 4, 5, 3),
              # several 256-column blocks and row tiles of the LDS-tile kernel, rows of whole 16-byte pieces for the
              # four-column gradient kernel (with and without padding), a stride whose tile does not fit LDS
              ((2, 1, 40, 1100), 5, 2, 0), ((1, 2, 30, 64), 3, 2, 1), ((1, 1, 24, 520), 2, 2, 0), ((1, 1, 20, 36), 7, 3, 2),
              ((1, 1, 40, 2000), 3, 20, 0)]


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


@pytest.mark.parametrize("shape,pool,stride,pad", POOL_CASES)
def test_avgpool_forward_and_backward_bit_exact(nz, oracle, shape, pool, stride, pad):
    rng = np.random.default_rng(sum(shape) + pool + stride)
    x = rng.uniform(-1, 1, shape).astype(np.float32)
    want = oracle.avgpool2d(x, pool, stride, pad)
    got = host(nz.avgpool2d(dev(x), pool, stride, pad))
    assert got.shape == want.shape and np.array_equal(got, want)
    dy = rng.uniform(-1, 1, want.shape).astype(np.float32)
    base = rng.uniform(-1, 1, shape).astype(np.float32)
    dx = dev(base)
    nz.avgpool2d_backward(dx, dev(dy), pool, stride, pad)
    assert np.array_equal(host(dx), oracle.avgpool2d_backward(base, dy, pool, stride, pad))


def _random_pool_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        pool, stride = int(rng.integers(1, 8)), int(rng.integers(1, 5))
        pad = int(rng.integers(0, pool))
        H, W = int(rng.integers(pool, 60)), int(rng.choice([8, 12, 16, 28, 31, 40, 64, 112, 300]))
        if W + 2 * pad < pool or H + 2 * pad < pool:
            continue
        cases.append(((int(rng.integers(1, 4)), int(rng.integers(1, 5)), H, W), pool, stride, pad))
    return cases


@pytest.mark.parametrize("shape,pool,stride,pad", _random_pool_cases(40, 11))
def test_avgpool_random_geometries_bit_exact(nz, oracle, shape, pool, stride, pad):
    rng = np.random.default_rng(sum(shape) * 3 + pool * 5 + stride * 7 + pad)
    x = rng.uniform(-1, 1, shape).astype(np.float32)
    want = oracle.avgpool2d(x, pool, stride, pad)
    assert np.array_equal(host(nz.avgpool2d(dev(x), pool, stride, pad)), want)
    dy = rng.uniform(-1, 1, want.shape).astype(np.float32)
    base = rng.uniform(-1, 1, shape).astype(np.float32)
    dx = dev(base)
    nz.avgpool2d_backward(dx, dev(dy), pool, stride, pad)
    assert np.array_equal(host(dx), oracle.avgpool2d_backward(base, dy, pool, stride, pad))
    # overwrite: the same sums started from zero, whatever dx held (NaN here: an old value that is read shows up)
    dx = dev(np.full(shape, np.nan, np.float32))
    nz.avgpool2d_backward(dx, dev(dy), pool, stride, pad, overwrite=True)
    assert np.array_equal(host(dx), oracle.avgpool2d_backward(np.zeros(shape, np.float32), dy, pool, stride, pad))


def test_avgpool_rejects_bad_geometry(nz):
    x = dev(np.zeros((1, 1, 4, 4)))
    with pytest.raises(nz.NzHipError):
        nz.avgpool2d(x, 5, 1, 0)                                   # window larger than the input
    with pytest.raises(nz.NzHipError):
        nz.avgpool2d(x, 2, 0, 0)                                   # zero stride
    with pytest.raises(nz.NzHipError):
        nz.avgpool2d_backward(x, dev(np.zeros((1, 1, 3, 3))), 2, 2, 0)   # dy extent does not match


def test_bce_loss_and_backward(nz, oracle):
    rng = np.random.default_rng(11)
    for n in (1, 7, 360, 4097, 300001):
        p = rng.uniform(0.1, 0.9, n).astype(np.float32)
        t = rng.uniform(0.1, 0.9, n).astype(np.float32)
        want = oracle.bce_loss(p, t)
        got = float(host(nz.bce_loss(dev(p), dev(t)))[0])
        p64, t64 = p.astype(np.float64), t.astype(np.float64)
        truth = float(np.mean(-t64 * np.log(p64) - (1 - t64) * np.log1p(-p64)))
        assert abs(got - truth) <= 1e-5 * truth and abs(want - truth) <= 1e-4 * truth, n
        assert np.array_equal(host(nz.bce_backward(dev(p), dev(t))), oracle.bce_backward(p, t)), n
    # the loss value does not depend on scheduling: the same input gives the same bits
    a = host(nz.bce_loss(dev(p), dev(t)))
    b = host(nz.bce_loss(dev(p), dev(t)))
    assert np.array_equal(a, b)


def test_mse_loss_and_backward(nz, oracle):
    rng = np.random.default_rng(13)
    for n in (1, 9, 360, 70001):
        p = rng.uniform(-2, 2, n).astype(np.float32)
        t = rng.uniform(-2, 2, n).astype(np.float32)
        truth = float(np.mean((p.astype(np.float64) - t.astype(np.float64)) ** 2))
        got = float(host(nz.mse_loss(dev(p), dev(t)))[0])
        assert abs(got - truth) <= 1e-5 * truth and abs(oracle.mse_loss(p, t) - truth) <= 1e-4 * truth, n
        assert np.array_equal(host(nz.mse_backward(dev(p), dev(t))), oracle.mse_backward(p, t)), n


def test_expand_and_compress_bit_exact(nz, oracle):
    rng = np.random.default_rng(12)
    x = rng.normal(size=(1, 3, 16, 5)).astype(np.float32)
    assert np.array_equal(host(nz.expand(dev(x), 7)), oracle.expand(x, 7))
    g = rng.normal(size=(7, 3, 16, 5)).astype(np.float32)
    base = rng.normal(size=(1, 3, 16, 5)).astype(np.float32)
    out = dev(base)
    nz.compress(out, dev(g))
    assert np.array_equal(host(out), oracle.compress(base, g))


def test_readme_network_sizes_through_size_independent_properties(nz):
    """The pooling and loss operators at the README network's sizes (10 x 1 x 1024 x 1024 -> 510 x 510), where the
    CPU oracle would take too long: a constant image stays constant, pooling and its gradient are adjoint
    (<pool(x), dy> = <x, pool^T(dy)>), the gradient hands out exactly what it receives (no padding), and the loss
    and its gradient agree with fp64 formulas evaluated by torch on the same data."""
    import torch
    gen = torch.Generator(device="cuda").manual_seed(21)
    x = torch.rand((10, 1, 1024, 1024), device="cuda", generator=gen)
    y = nz.avgpool2d(x, 5, 2, 0)
    assert tuple(y.shape) == (10, 1, 510, 510)
    const = nz.avgpool2d(torch.full_like(x, 0.375), 5, 2, 0)              # 0.375 * 25 and / 25 are exact
    assert bool((const == 0.375).all())
    dy = torch.rand(y.shape, device="cuda", generator=gen) - 0.5
    dx = torch.zeros_like(x)
    nz.avgpool2d_backward(dx, dy, 5, 2, 0)
    lhs = float((y.double() * dy.double()).sum())
    rhs = float((x.double() * dx.double()).sum())
    assert abs(lhs - rhs) <= 1e-5 * max(1.0, abs(lhs))
    assert abs(float(dx.double().sum()) - float(dy.double().sum())) <= 1e-4 * max(1.0, abs(float(dy.double().sum())))
    # torch's own pooling (count_include_pad irrelevant without padding) as a third opinion on the values
    ref = torch.nn.functional.avg_pool2d(x.double(), 5, 2).float()
    assert float((y - ref).abs().max()) <= 2e-6
    p = torch.rand(10 * 1024 * 1024, device="cuda", generator=gen) * 0.8 + 0.1
    t = torch.rand(p.shape, device="cuda", generator=gen) * 0.8 + 0.1
    truth = float((-(t.double()) * torch.log(p.double()) - (1 - t.double()) * torch.log1p(-p.double())).mean())
    assert abs(float(nz.bce_loss(p, t)[0]) - truth) <= 1e-5 * truth
    g = nz.bce_backward(p, t)
    gt = ((p.double() - t.double()) / (p.double() * (1 - p.double())) / p.numel())
    assert float(((g.double() - gt).abs() / gt.abs().clamp_min(1e-12)).max()) <= 1e-5
    mse_truth = float(((p.double() - t.double()) ** 2).mean())
    assert abs(float(nz.mse_loss(p, t)[0]) - mse_truth) <= 1e-5 * mse_truth

