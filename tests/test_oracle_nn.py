"""Pins the oracle's average pooling, binary cross-entropy and expand / compress: against independent
formulations (windows taken with numpy's sliding views over a NaN-padded image, the adjoint identity
between pooling and its gradient, finite differences of the loss) and closed forms. The reference's
tests hold loop nests over random data and no literal vectors for these operators
(test/Test.cpp:3179-3246, 3316-3385, 1937-1999, 2663-2730)."""
import numpy as np
import pytest

POOL_CASES = [((2, 3, 4, 5), 2, 2, 0),        # the reference test's shape (Test.cpp:3180-3187)
              ((1, 2, 9, 7), 3, 1, 1), ((2, 1, 10, 10), 5, 2, 0), ((1, 1, 6, 8), 4, 3, 2), ((1, 3, 5, 5), 5, 1, 2),
              ((2, 2, 7, 3), 1, 1, 0), ((1, 1, 8, 8), 3, 2, 1)]


def windows_mean(x, pool, stride, pad):
    """Mean over the in-image cells of every window, through a NaN-padded copy and sliding views."""
    xp = np.pad(x.astype(np.float64), ((0, 0), (0, 0), (pad, pad), (pad, pad)), constant_values=np.nan)
    v = np.lib.stride_tricks.sliding_window_view(xp, (pool, pool), axis=(2, 3))[:, :, ::stride, ::stride]
    cnt = np.sum(~np.isnan(v), axis=(4, 5))
    return np.where(cnt > 0, np.nansum(v, axis=(4, 5)) / np.maximum(cnt, 1), 0.0), cnt


@pytest.mark.parametrize("shape,pool,stride,pad", POOL_CASES)
def test_avgpool_matches_sliding_windows(oracle, shape, pool, stride, pad):
    rng = np.random.default_rng(sum(shape) + pool)
    x = rng.uniform(0.1, 0.9, shape).astype(np.float32)
    got = oracle.avgpool2d(x, pool, stride, pad)
    want, _ = windows_mean(x, pool, stride, pad)
    assert got.shape == want.shape
    assert np.allclose(got, want, rtol=2e-6, atol=0)
    # integers: every sum is exact in fp32, so the only rounding is the one division
    xi = rng.integers(-20, 21, shape).astype(np.float32)
    wi, cnt = windows_mean(xi, pool, stride, pad)
    sums = np.rint(wi * cnt)
    assert np.array_equal(oracle.avgpool2d(xi, pool, stride, pad), (sums.astype(np.float32) / cnt.astype(np.float32)))
    # a constant image stays constant whatever the padding (cells in the padding do not count)
    assert np.array_equal(oracle.avgpool2d(np.full(shape, 3.0, np.float32), pool, stride, pad),
                          np.full(got.shape, 3.0, np.float32))


def test_avgpool_identity_window(oracle):
    x = np.random.default_rng(3).normal(size=(2, 2, 5, 6)).astype(np.float32)
    assert np.array_equal(oracle.avgpool2d(x, 1, 1, 0), x)


@pytest.mark.parametrize("shape,pool,stride,pad", POOL_CASES)
def test_avgpool_backward_is_the_adjoint_and_accumulates(oracle, shape, pool, stride, pad):
    rng = np.random.default_rng(sum(shape) + 7 * pool)
    x = rng.normal(size=shape).astype(np.float32)
    y = oracle.avgpool2d(x, pool, stride, pad)
    dy = rng.normal(size=y.shape).astype(np.float32)
    dx = oracle.avgpool2d_backward(np.zeros(shape, np.float32), dy, pool, stride, pad)
    # <pool(x), dy> = <x, pool^T(dy)>: holds with and without padding because the forward divides by the same count
    lhs = float((y.astype(np.float64) * dy).sum()), float((x.astype(np.float64) * dx).sum())
    assert abs(lhs[0] - lhs[1]) <= 1e-4 * max(1.0, abs(lhs[0]))
    base = rng.normal(size=shape).astype(np.float32)
    acc = oracle.avgpool2d_backward(base, dy, pool, stride, pad)
    assert np.allclose(acc, base + dx, rtol=1e-5, atol=1e-6)      # din += ..., not din = ...
    # every output cell hands out exactly its gradient when no window cell lies in the padding
    if pad == 0:
        assert np.isclose(dx.astype(np.float64).sum(), dy.astype(np.float64).sum(), rtol=1e-5, atol=1e-5)


def test_bce_loss_and_gradient(oracle):
    rng = np.random.default_rng(5)
    p = rng.uniform(0.1, 0.9, (2, 3, 12, 5)).astype(np.float32)       # the reference test's shape (Test.cpp:1938-1941)
    t = rng.uniform(0.1, 0.9, p.shape).astype(np.float32)
    p64, t64 = p.astype(np.float64), t.astype(np.float64)
    want = float(np.mean(-t64 * np.log(p64) - (1 - t64) * np.log1p(-p64)))
    assert abs(oracle.bce_loss(p, t) - want) <= 1e-5 * want
    assert abs(oracle.bce_loss(np.full(8, 0.5, np.float32), np.full(8, 0.5, np.float32)) - np.log(2.0)) < 1e-6
    # perfect confident predictions cost nothing, whatever the label
    assert oracle.bce_loss(np.array([1.0 - 1e-7, 1e-7], np.float32), np.array([1.0, 0.0], np.float32)) < 1e-6
    g = oracle.bce_backward(p, t)
    # central differences of the float64 loss
    eps = 1e-6
    for idx in [(0, 0, 0, 0), (1, 2, 11, 4), (0, 1, 5, 3)]:
        hi, lo = p64.copy(), p64.copy()
        hi[idx] += eps
        lo[idx] -= eps
        f = lambda q: np.mean(-t64 * np.log(q) - (1 - t64) * np.log1p(-q))
        assert abs(g[idx] - (f(hi) - f(lo)) / (2 * eps)) <= 1e-4 * abs(g[idx]) + 1e-7
    assert np.allclose(g, ((p64 - t64) / (p64 * (1 - p64)) / p.size), rtol=1e-6, atol=0)
    # the gradient vanishes where the prediction equals the label
    assert np.array_equal(oracle.bce_backward(t, t), np.zeros_like(t))


def test_mse_loss_and_gradient(oracle):
    rng = np.random.default_rng(8)
    p = rng.uniform(0.1, 0.9, (2, 3, 12, 5)).astype(np.float32)       # the reference test's shape (Test.cpp:1873-1876)
    t = rng.uniform(0.1, 0.9, p.shape).astype(np.float32)
    p64, t64 = p.astype(np.float64), t.astype(np.float64)
    want = float(np.mean((p64 - t64) ** 2))
    assert abs(oracle.mse_loss(p, t) - want) <= 1e-5 * want
    assert oracle.mse_loss(t, t) == 0.0
    assert abs(oracle.mse_loss(np.full(7, 3.0, np.float32), np.full(7, 1.0, np.float32)) - 4.0) < 1e-6
    g = oracle.mse_backward(p, t)
    assert np.allclose(g, 2 * (p64 - t64) / p.size, rtol=1e-6, atol=0)
    # the loss is quadratic: its gradient is exact under central differences
    hi, lo = p64.copy(), p64.copy()
    hi[1, 2, 3, 4] += 1e-3
    lo[1, 2, 3, 4] -= 1e-3
    fd = (np.mean((hi - t64) ** 2) - np.mean((lo - t64) ** 2)) / 2e-3
    assert abs(g[1, 2, 3, 4] - fd) <= 1e-5 * abs(fd)


def test_expand_and_compress(oracle):
    rng = np.random.default_rng(6)
    x = rng.integers(-9, 10, (1, 2, 3, 4)).astype(np.float32)
    e = oracle.expand(x, 5)
    assert e.shape == (5, 2, 3, 4) and np.array_equal(e, np.broadcast_to(x, (5, 2, 3, 4)))
    g = rng.integers(-9, 10, (5, 2, 3, 4)).astype(np.float32)
    base = rng.integers(-9, 10, (1, 2, 3, 4)).astype(np.float32)
    assert np.array_equal(oracle.compress(base, g), base + g.sum(axis=0, keepdims=True))
