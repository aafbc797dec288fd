"""Prepared-operand handles (nzhip_prepared): the fp16 image of a weight operand kept between calls. Results must be
bit-identical with and without a handle; the image is built once per operand, rebuilt when the operand, the shape or
the route changes and after nzhip_prepared_invalidate; routes without an image ignore the handle."""
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


def rnd(shape, seed, scale=1.0):
    import torch
    g = torch.Generator(device="cpu").manual_seed(seed)
    return ((torch.rand(shape, generator=g) * 2 - 1) * scale).cuda()


@pytest.mark.parametrize("M,K,N,b_trans", [(4096, 1024, 4096, True), (3072, 768, 3072, False), (2000, 800, 2000, True)])
def test_gemm_with_a_prepared_b_image(nz, M, K, N, b_trans):
    import torch
    A, A2 = rnd((M, K), 1), rnd((M, K), 2)
    B = rnd((N, K) if b_trans else (K, N), 3)
    bias = rnd((N,), 4)
    kw = dict(b_trans=b_trans, bias=bias, bias_strides=(0, 1), relu=True)
    want, want2 = nz.gemm(A, B, **kw), nz.gemm(A2, B, **kw)
    h = nz.Prepared()
    try:
        assert torch.equal(nz.gemm(A, B, prepared_b=h, **kw), want) and h.fills() == 1
        assert torch.equal(nz.gemm(A2, B, prepared_b=h, **kw), want2) and h.fills() == 1     # B's image reused
        # the weights change in place: without invalidation the OLD product comes back (documented), with it the new one
        B.mul_(0.5)
        new = nz.gemm(A, B, **kw)
        assert torch.equal(nz.gemm(A, B, prepared_b=h, **kw), want)
        h.invalidate()
        assert torch.equal(nz.gemm(A, B, prepared_b=h, **kw), new) and h.fills() == 2
        # another operand behind the same handle: rebuilt by itself
        B3 = rnd(tuple(B.shape), 5)
        assert torch.equal(nz.gemm(A, B3, prepared_b=h, **kw), nz.gemm(A, B3, **kw)) and h.fills() == 3
        # a route without an image (a skinny product) ignores the handle
        a1 = rnd((1, K), 6)
        assert torch.equal(nz.gemm(a1, B3, prepared_b=h, b_trans=b_trans), nz.gemm(a1, B3, b_trans=b_trans)) and h.fills() == 3
    finally:
        h.close()


CONVS = [  # N, C, H, W, O, K, pad, w_batch: double-buffer resident kernel, single-buffer resident kernel, slab kernel, ...,
    # and the any-geometry kernel (5x5)
    (4, 64, 64, 64, 128, 3, 1, 1), (2, 48, 40, 72, 64, 3, 1, 1), (2, 24, 33, 47, 40, 3, 1, 1), (8, 160, 64, 64, 128, 3, 1, 1),
    (3, 24, 20, 20, 48, 1, 0, 1), (8, 16, 64, 64, 32, 3, 1, 8), (16, 16, 32, 32, 16, 5, 2, 1)]   # (1x1 below 32 channels: from there on it is a plain product without an image)


@pytest.mark.parametrize("N,C,H,W,O,K,pad,wb", CONVS)
def test_conv_forward_with_prepared_weights(nz, N, C, H, W, O, K, pad, wb):
    import torch
    x, x2 = rnd((N, C, H, W), 11), rnd((N, C, H, W), 12)
    w = rnd((wb, 1, C * K * K, O), 13, 0.1)
    bias = rnd((O,), 14)
    kw = dict(bias_strides=(0, 1), relu=True)
    want, want2 = nz.conv2d_forward(x, w, bias, K, K, 1, pad, **kw), nz.conv2d_forward(x2, w, bias, K, K, 1, pad, **kw)
    h = nz.Prepared()
    try:
        assert torch.equal(nz.conv2d_forward(x, w, bias, K, K, 1, pad, prepared_w=h, **kw), want)
        first = h.fills()
        assert first == 1
        assert torch.equal(nz.conv2d_forward(x2, w, bias, K, K, 1, pad, prepared_w=h, **kw), want2) and h.fills() == 1
        w.mul_(-1.5)
        new = nz.conv2d_forward(x, w, bias, K, K, 1, pad, **kw)
        h.invalidate()
        assert torch.equal(nz.conv2d_forward(x, w, bias, K, K, 1, pad, prepared_w=h, **kw), new) and h.fills() == 2
    finally:
        h.close()


def test_conv_routes_without_an_image_ignore_the_handle(nz):
    # the row-streaming kernel for a handful of channels, and the column-matrix route of a layer with few patches on
    # images so small that the any-geometry kernel's segments would be three quarters empty
    import torch
    h = nz.Prepared()
    try:
        for xs, ws in (((2, 3, 64, 64), (1, 1, 27, 1)), ((4, 512, 8, 8), (1, 1, 512 * 9, 256))):
            x, w = rnd(xs, 21), rnd(ws, 22, 0.05)
            got = nz.conv2d_forward(x, w, None, 3, 3, 1, 1, prepared_w=h)
            assert torch.equal(got, nz.conv2d_forward(x, w, None, 3, 3, 1, 1)) and h.fills() == 0
    finally:
        h.close()


def test_a_handle_moves_between_gemm_and_conv(nz):
    # one handle, used first for a GEMM operand and then for convolution weights: the image is rebuilt, never mixed up
    import torch
    A, B = rnd((2048, 1024), 31), rnd((2048, 1024), 32)
    x, w = rnd((2, 64, 32, 64), 33), rnd((1, 1, 576, 128), 34, 0.1)
    h = nz.Prepared()
    try:
        assert torch.equal(nz.gemm(A, B, b_trans=True, prepared_b=h, force_tile=0), nz.gemm(A, B, b_trans=True))
        n1 = h.fills()
        assert torch.equal(nz.conv2d_forward(x, w, None, 3, 3, 1, 1, prepared_w=h), nz.conv2d_forward(x, w, None, 3, 3, 1, 1))
        assert h.fills() == n1 + 1
        assert torch.equal(nz.gemm(A, B, b_trans=True, prepared_b=h), nz.gemm(A, B, b_trans=True))
    finally:
        h.close()
