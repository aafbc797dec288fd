"""Parity of the conv lowering (im2col, col2im, fused Conv2d forward) on the GPU with the CPU
oracle; called through the C-ABI.  Integer-valued cases must match bit for bit; float cases
meet max-rel <= 1e-3 / Frobenius-rel <= 1e-4 against the fp64 direct convolution of the same
fp16-rounded operands (max-rel floored at the RMS of the truth)."""
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


IM2COL_CASES = [((2, 3, 4, 5), 3, 3, 1, 1), ((1, 1, 1, 1), 1, 1, 1, 0), ((2, 2, 7, 6), 3, 2, 2, 0),
                ((1, 3, 8, 9), 2, 4, 2, 2), ((3, 1, 5, 5), 5, 5, 1, 2), ((2, 4, 6, 6), 1, 1, 3, 0),
                ((2, 5, 33, 47), 3, 3, 1, 1),
                # stride 1 with C*K_h*K_w a multiple of 4: the kernel that stages input rows in LDS (64-pixel segments,
                # 32-channel chunks with a tail, compile-time and run-time kernel extents)
                ((2, 4, 6, 7), 3, 3, 1, 1), ((1, 64, 5, 130), 3, 3, 1, 1), ((2, 40, 9, 70), 3, 3, 1, 0),
                ((2, 8, 7, 66), 1, 1, 1, 0), ((1, 4, 9, 75), 5, 5, 1, 2), ((2, 2, 8, 9), 2, 2, 1, 1), ((1, 36, 4, 64), 3, 3, 1, 2),
                # narrow images: several whole output rows per workgroup (4 rows of 16, 9 of 7 with a 7-row tail image,
                # 2 of 30 with an odd row count, one pixel per row, pad 0 so that the output is narrower than the input)
                ((2, 40, 16, 16), 3, 3, 1, 1), ((3, 12, 7, 7), 3, 3, 1, 1), ((1, 8, 5, 30), 3, 3, 1, 1),
                ((2, 4, 9, 1), 3, 3, 1, 1), ((2, 16, 12, 12), 5, 5, 1, 0), ((1, 68, 14, 14), 1, 1, 1, 0),
                # other strides with a multiple of 4: the 16-byte store variant of the per-element kernel
                ((2, 4, 9, 9), 3, 3, 2, 1), ((1, 8, 10, 12), 2, 3, 3, 0)]


@pytest.mark.parametrize("shape,k_h,k_w,stride,pad", IM2COL_CASES)
def test_im2col_bit_exact(nz, oracle, shape, k_h, k_w, stride, pad):
    x = np.random.default_rng(sum(shape)).uniform(0.1, 0.9, size=shape).astype(np.float32)
    assert np.array_equal(host(nz.im2col(dev(x), k_h, k_w, stride, pad)), oracle.im2col(x, k_h, k_w, stride, pad))


@pytest.mark.parametrize("n,c,h,w", [(2, 3, 4, 5), (1, 1, 1, 1), (3, 40, 9, 11), (2, 128, 16, 16), (1, 1, 50, 70), (3, 7, 1, 1)])
def test_col2im_bit_exact(nz, oracle, n, c, h, w):
    col = np.random.default_rng(n + c + h + w).uniform(-1, 1, size=(n, 1, h * w, c)).astype(np.float32)
    assert np.array_equal(host(nz.col2im(dev(col), h, w)), oracle.col2im(col, h, w))


def test_add_broadcast_bit_exact(nz, oracle):
    rng = np.random.default_rng(2)
    for sa, sb in [((2, 3, 4, 4), (1, 1, 4, 4)), ((2, 3, 5, 3), (1, 3, 5, 3)), ((1, 3, 5, 3), (2, 1, 5, 3)),
                   ((4, 1, 64, 1), (1, 1, 64, 1)), ((3, 1, 30, 7), (1, 1, 30, 7))]:
        a = rng.normal(size=sa).astype(np.float32)
        b = rng.normal(size=sb).astype(np.float32)
        assert np.array_equal(host(nz.add_broadcast(dev(a), dev(b))), oracle.matrix_add(a, b))
    with pytest.raises(nz.NzHipError) as ei:
        nz.add_broadcast(dev(np.zeros((2, 1, 3, 3))), dev(np.zeros((3, 1, 3, 3))))
    assert ei.value.status == -2 and "not broadcast compatible" in ei.value.message


CONV_CASES = [
    # N, C, H, W, O, k_h, k_w, stride, pad, w_batch
    (2, 3, 6, 7, 4, 3, 3, 1, 1, 1),
    (2, 3, 6, 7, 4, 3, 3, 1, 1, 2),
    (1, 2, 9, 8, 3, 2, 3, 2, 0, 1),
    (3, 1, 5, 5, 1, 3, 3, 1, 2, 1),
    (2, 16, 20, 24, 40, 3, 3, 1, 1, 1),
    (1, 3, 40, 64, 1, 3, 3, 1, 1, 1),
    (2, 8, 17, 19, 5, 5, 5, 2, 2, 1),
    (1, 70, 9, 9, 130, 1, 1, 1, 0, 1),
    (2, 130, 9, 12, 70, 1, 1, 1, 0, 1),     # 1x1 with 128 or more input channels: one batched product
    (2, 160, 8, 8, 40, 1, 1, 1, 0, 2),      # ... with per-sample weights
    (2, 200, 5, 5, 16, 1, 1, 1, 0, 1),      # ... tiny images and fewer outputs than inputs: a product as well
    (2, 24, 9, 11, 40, 1, 1, 2, 0, 1),      # 1x1 with a stride: every second pixel gathered, then the 1x1 stride-1 kernels
    (3, 130, 7, 13, 20, 1, 1, 3, 0, 3),     # ... stride 3, odd extents, per-sample weights, as a batched product
    (2, 24, 40, 70, 9, 3, 3, 1, 0, 1),      # no padding, ragged width (scalar staging path)
    (1, 9, 33, 36, 140, 3, 3, 1, 2, 1),     # padding 2: both halo columns on the left
    (2, 20, 16, 64, 64, 3, 3, 1, 1, 2),     # per-sample weights
    (1, 16, 12, 40, 8, 3, 3, 1, 3, 1),      # padding larger than the kernel reach: workspace route
    (3, 20, 6, 6, 80, 3, 3, 1, 1, 3),       # per-sample weights, output pixels x 2 <= output channels: the column matrix instead of a weight image per copy
    (4, 33, 5, 7, 130, 5, 5, 1, 2, 4),      # ... 5x5, two channel tiles' worth of outputs
    # resident weights with two halo buffers (64 channels -> 128-channel tile, 128 -> 64-channel tile, 64-wide patches)
    (1, 64, 9, 64, 128, 3, 3, 1, 1, 1),     # rows not a multiple of the 4-row patch
    (2, 50, 12, 72, 100, 3, 3, 1, 1, 1),    # last chunk with 2 of 16 channels, part of a channel tile, ragged second patch
    (1, 64, 8, 68, 130, 3, 3, 1, 0, 1),     # no padding, two channel tiles (the second with 2 channels)
    (1, 64, 6, 64, 128, 3, 3, 1, 2, 1),     # padding 2
    (2, 128, 10, 64, 64, 3, 3, 1, 1, 1),    # eight chunks, 64-channel tile
    (1, 120, 7, 128, 40, 3, 3, 1, 1, 1),    # eight chunks, the last partial, 40 of 64 channels
    (33, 64, 32, 64, 128, 3, 3, 1, 1, 1),   # 264 patches for 256 workgroups: uneven patch counts
    (2, 32, 10, 64, 128, 3, 3, 1, 1, 1),    # two chunks, 128-channel tile
    (1, 20, 9, 72, 100, 3, 3, 1, 1, 1),     # two chunks, the second with 4 of 16 channels, part of a channel tile
    (2, 64, 10, 64, 64, 3, 3, 1, 1, 1),     # four chunks, 64-channel tile
    (1, 30, 7, 128, 40, 3, 3, 1, 0, 1),     # two chunks, 64-channel tile, no padding
    (3, 17, 5, 64, 200, 3, 3, 1, 2, 1),     # two chunks (1 channel in the second), two channel tiles, padding 2
]


@pytest.mark.parametrize("N,C,H,W,O,k_h,k_w,stride,pad,w_batch", CONV_CASES)
def test_conv2d_integers_bit_exact(nz, oracle, N, C, H, W, O, k_h, k_w, stride, pad, w_batch):
    rng = np.random.default_rng(N + C + H + W + O + k_h)
    x = rng.integers(-4, 5, size=(N, C, H, W)).astype(np.float32)
    w = rng.integers(-3, 4, size=(O, C, k_h, k_w)).astype(np.float32)
    bias = rng.integers(-2, 3, size=(O,)).astype(np.float32)
    w_ref = oracle.weights_oihw_to_ref(w)
    if w_batch > 1:
        w_ref = np.ascontiguousarray(np.broadcast_to(w_ref, (w_batch,) + w_ref.shape[1:]))
    truth = oracle.conv2d_direct_f64(x, w, bias, stride, pad, relu=True)
    got = host(nz.conv2d_forward(dev(x), dev(w_ref), dev(bias), k_h, k_w, stride, pad, bias_strides=(0, 1), relu=True))
    assert np.array_equal(got.astype(np.float64), truth)
    # the unfused graph, node by node (src/Model.cu:244-263), gives the same numbers
    Ho, Wo = oracle.out_hw(H, W, k_h, k_w, stride, pad)
    col = nz.im2col(dev(x), k_h, k_w, stride, pad)
    res = nz.tensorcore_gemm(col, dev(w_ref))
    res = nz.add_broadcast(res, dev(oracle.bias_channel_to_ref(bias, Ho * Wo)))
    y = nz.relu(nz.col2im(res, Ho, Wo))
    assert np.array_equal(host(y), got)


CONV_ANY_GEOMETRY = [  # N, C, H, W, O, k_h, k_w, stride, pad, w_batch, per-pixel bias: enough 256-pixel segments for the
    # implicit-GEMM kernel that takes any kernel extent and stride (rows that allow 16-byte loads)
    (16, 16, 32, 32, 16, 5, 5, 1, 2, 1, False),     # 5x5, 32-wide segments of 8 rows, 64-channel tile
    (32, 24, 33, 64, 70, 3, 3, 2, 1, 1, False),     # stride 2, two chunks (the second half empty), 70 channels in two 64-channel tiles
    (256, 8, 32, 32, 70, 3, 3, 2, 1, 1, False),     # a workgroup for every compute unit: 128-channel tile with 70 channels
    (64, 8, 32, 32, 65, 5, 5, 1, 2, 1, False),      # the same tile with one staging task per thread ...
    (64, 8, 48, 192, 65, 3, 3, 3, 1, 1, False),     # ... and with three
    (16, 16, 48, 192, 8, 3, 3, 3, 1, 1, False),     # stride 3: three staging tasks per thread
    (4, 8, 66, 260, 9, 3, 3, 2, 1, 1, False),       # 130 output columns: one row per segment, the second half of it empty
    (40, 40, 20, 24, 130, 2, 3, 2, 0, 40, False),   # 2x3 kernel, no padding, per-sample weights, two channel tiles
    (32, 32, 30, 40, 64, 5, 5, 2, 3, 1, True),      # padding 3, per-pixel bias (turned into channel planes first)
    (64, 16, 14, 16, 32, 3, 3, 2, 1, 1, False),     # 7 x 8 outputs: a 16 x 16 segment would be less than half full, column matrix
    (32, 16, 24, 32, 32, 3, 3, 2, 1, 1, False),     # 12 x 16 outputs: a segment spans the whole image and more
    (4, 16, 40, 128, 16, 5, 5, 4, 2, 1, False),     # stride 4 with 128-wide... the tile does not fit a thread's staging share: column matrix
    # few segments and many channels: the contraction split over groups of channel chunks, the groups' sums added by a
    # second kernel (a 3x3 stride-1 layer whose weights are beyond LDS, and a 5x5 stride-2 one)
    (16, 256, 16, 16, 64, 3, 3, 1, 1, 1, False),
    (24, 96, 32, 32, 32, 5, 5, 2, 2, 1, True),
    # rows that are not whole 16-byte pieces (14- and 30-wide images): staging with per-column bounds
    (64, 16, 14, 14, 32, 5, 5, 1, 2, 1, False),
    (64, 24, 21, 30, 70, 3, 3, 2, 1, 1, True),
    (16, 256, 14, 14, 96, 3, 3, 1, 1, 1, False),    # ... with the contraction split (a 3x3 stride-1 layer, weights beyond LDS)
    # fewer than eight input channels (a network's first layer): one chunk, most of it zero
    (8, 3, 64, 64, 64, 3, 3, 1, 1, 1, True),        # RGB, 3x3 stride 1, the reference's per-pixel bias
    (32, 1, 28, 28, 6, 5, 5, 1, 0, 1, False),       # one channel, 5x5 without padding, six output channels
    (8, 3, 96, 96, 20, 7, 7, 2, 3, 1, False),       # 7x7 stride 2: the slab of 49 taps beside a 13-row halo
    (6, 3, 50, 224, 64, 7, 7, 2, 3, 1, False),      # ... on 112 output columns: 128-wide segments do not fit, 4 x 64 pixels do
    (16, 5, 30, 30, 9, 3, 3, 1, 1, 16, False),      # rows that are not whole 16-byte pieces, per-sample weights
    # two chunks per loop step (at least four chunks, contraction not split, rows of whole 16-byte pieces): both channel
    # tiles with one, two and three staging tasks per thread, with and without the per-pixel bias, an odd number of
    # chunks (the step's second slab is zero) and a 3x3 stride-1 layer with 192 channels, which takes this kernel
    (256, 64, 16, 16, 48, 5, 5, 1, 2, 1, False), (256, 80, 16, 16, 48, 5, 5, 1, 2, 1, True),
    (16, 192, 32, 128, 40, 3, 3, 1, 1, 1, True), (128, 64, 32, 64, 24, 3, 3, 2, 1, 1, False),
    (256, 192, 16, 16, 70, 3, 3, 1, 1, 1, False), (256, 200, 16, 16, 70, 3, 3, 1, 1, 1, True),
    (16, 192, 32, 128, 130, 3, 3, 1, 1, 1, False), (128, 72, 32, 64, 70, 3, 3, 2, 1, 1, True),
    # the per-pixel bias on the 128-channel tile and with two and three staging tasks per thread
    (64, 8, 32, 32, 65, 5, 5, 1, 2, 1, True),
    (256, 8, 32, 32, 70, 3, 3, 2, 1, 1, True),
    (16, 16, 48, 192, 8, 3, 3, 3, 1, 1, True),
]


@pytest.mark.parametrize("N,C,H,W,O,k_h,k_w,stride,pad,w_batch,pix", CONV_ANY_GEOMETRY)
def test_conv2d_any_geometry_integers_bit_exact(nz, oracle, N, C, H, W, O, k_h, k_w, stride, pad, w_batch, pix):
    rng = np.random.default_rng(N * 3 + C * 5 + H * 7 + W * 11 + O * 13 + k_h + stride)
    Ho, Wo = oracle.out_hw(H, W, k_h, k_w, stride, pad)
    x = rng.integers(-4, 5, size=(N, C, H, W)).astype(np.float32)
    ws = [rng.integers(-3, 4, size=(O, C, k_h, k_w)).astype(np.float32) for _ in range(w_batch)]
    w_ref = np.concatenate([oracle.weights_oihw_to_ref(w) for w in ws], axis=0)
    if pix:
        bias = rng.integers(-2, 3, size=(1, 1, Ho * Wo, O)).astype(np.float32)
        strides, badd = (O, 1), bias.reshape(Ho, Wo, O).transpose(2, 0, 1)[None].astype(np.float64)
    else:
        bias = rng.integers(-2, 3, size=(O,)).astype(np.float32)
        strides, badd = (0, 1), bias.reshape(1, O, 1, 1).astype(np.float64)
    got = host(nz.conv2d_forward(dev(x), dev(w_ref), dev(bias), k_h, k_w, stride, pad, bias_strides=strides, relu=True))
    for n in range(N):
        w = ws[n if w_batch > 1 else 0]
        truth = np.maximum(oracle.conv2d_direct_f64(x[n:n + 1], w, None, stride, pad) + badd, 0)
        assert np.array_equal(got[n:n + 1].astype(np.float64), truth), (n,)


WIDENED = [  # N, C, H, W, O, k, stride, pad, w_batch, per-pixel bias: rows that are not whole 16-byte pieces on the any-geometry kernel
    # (5x5; stride 2 with the per-pixel bias; a split contraction; per-sample weights; two chunks per loop step, which such
    # rows only reach through the copy; 7x7 stride 2 on three channels)
    (64, 16, 14, 14, 32, 5, 1, 2, 1, False), (64, 24, 21, 30, 70, 3, 2, 1, 1, True), (16, 256, 14, 14, 96, 3, 1, 1, 1, False),
    (16, 5, 30, 30, 9, 3, 1, 1, 16, False), (256, 64, 14, 14, 48, 5, 1, 2, 1, False), (8, 3, 97, 97, 20, 7, 2, 3, 1, False),
    # 1x1 layers as products: planes of 49, 35 and 1225 pixels widened to 52, 36 and 1228 (shared and per-sample weights,
    # per-channel and per-pixel bias)
    (8, 130, 7, 7, 140, 1, 1, 0, 1, False), (6, 128, 5, 7, 130, 1, 1, 0, 6, True), (2, 136, 35, 35, 20, 1, 1, 0, 1, False)]


@pytest.mark.parametrize("N,C,H,W,O,k,stride,pad,w_batch,pix", WIDENED)
def test_conv2d_on_rows_widened_to_16_byte_pieces_is_bit_exact(nz, oracle, monkeypatch, N, C, H, W, O, k, stride, pad, w_batch, pix):
    # Large layers with such rows run on a zero-filled copy whose rows are the next multiple of 4 wide; the library reads
    # NZHIP_CONV_WIDEN per call, so the copy can be forced for shapes an oracle finishes quickly. Forward, and the
    # stride-1 data gradient (the same kernel on the output gradient, mirrored weights, accumulating in place).
    monkeypatch.setenv("NZHIP_CONV_WIDEN", "1")
    rng = np.random.default_rng(N * 3 + C * 5 + H * 7 + W * 11 + O * 13 + k + stride)
    Ho, Wo = oracle.out_hw(H, W, k, k, stride, pad)
    x = rng.integers(-4, 5, size=(N, C, H, W)).astype(np.float32)
    ws = [rng.integers(-3, 4, size=(O, C, k, k)).astype(np.float32) for _ in range(w_batch)]
    w_ref = np.concatenate([oracle.weights_oihw_to_ref(w) for w in ws], axis=0)
    if pix:
        bias = rng.integers(-2, 3, size=(1, 1, Ho * Wo, O)).astype(np.float32)
        strides, badd = (O, 1), bias.reshape(Ho, Wo, O).transpose(2, 0, 1)[None].astype(np.float64)
    else:
        bias = rng.integers(-2, 3, size=(O,)).astype(np.float32)
        strides, badd = (0, 1), bias.reshape(1, O, 1, 1).astype(np.float64)
    got = host(nz.conv2d_forward(dev(x), dev(w_ref), dev(bias), k, k, stride, pad, bias_strides=strides, relu=True))
    for n in range(N):
        w = ws[n if w_batch > 1 else 0]
        truth = np.maximum(oracle.conv2d_direct_f64(x[n:n + 1], w, None, stride, pad) + badd, 0)
        assert np.array_equal(got[n:n + 1].astype(np.float64), truth), ("forward", n)
    if stride == 1:
        dy = rng.integers(-4, 5, size=(N, O, Ho, Wo)).astype(np.float32)
        dx0 = rng.integers(-3, 4, size=(N, C, H, W)).astype(np.float32)
        for accumulate in (False, True):
            expect = oracle.conv2d_backward_data(dx0.copy() if accumulate else np.zeros_like(dx0), dy, w_ref, k, k, pad)
            got_dx = host(nz.conv2d_backward_data(dev(dx0), dev(dy), dev(w_ref), k, k, 1, pad, accumulate=accumulate))
            assert np.array_equal(got_dx, expect), ("data gradient", accumulate)


PER_SAMPLE = [  # N, C, H, W, O, k, pad, per-pixel bias: one weight copy per image, every copy different
    (4, 32, 12, 64, 128, 3, 1, False),    # two halo buffers, 128-channel tile, 64 workgroups per image
    (3, 64, 9, 64, 64, 3, 1, True),       # two halo buffers, 64-channel tile, per-pixel bias; 255 of 256 workgroups used
    (16, 64, 16, 64, 128, 3, 1, False),   # sixteen images, 16 workgroups each
    (5, 48, 10, 72, 100, 3, 1, False),    # three chunks: the single-buffer resident kernel
    (2, 64, 8, 64, 128, 3, 1, True),      # per-pixel bias with a 128-channel tile: the single-buffer resident kernel
    (6, 40, 9, 40, 70, 1, 0, False),      # 1x1, 32-wide patches, two channel tiles
    (3, 128, 9, 12, 24, 1, 0, True),      # 1x1 as a batched product, per-pixel bias as its bias matrix
    (2, 160, 8, 64, 128, 3, 1, False),    # weights beyond LDS: the per-patch slab kernel
    (300, 16, 4, 32, 16, 3, 1, False),    # more images than workgroups: the per-patch slab kernel
]


BIAS_SHARED_BY_IMAGES = [  # N, C, H, W, O, per-sample weights: a per-pixel bias on the resident kernels with a patch count per image
    # that is a multiple of 8, where every XCD takes the same eighth of all images (both halo-buffer variants, both
    # channel tiles, three images in a grid of 24, sixteen images with two workgroups per XCD each)
    (2, 32, 32, 64, 64, False), (2, 32, 32, 64, 64, True), (4, 64, 16, 128, 128, False), (4, 64, 16, 128, 128, True),
    (3, 64, 32, 64, 128, False), (16, 48, 32, 64, 100, True), (16, 64, 32, 128, 128, True), (5, 16, 64, 64, 40, False)]


@pytest.mark.parametrize("N,C,H,W,O,per_sample", BIAS_SHARED_BY_IMAGES)
def test_conv2d_per_pixel_bias_with_every_xcd_on_one_eighth_of_all_images(nz, oracle, N, C, H, W, O, per_sample):
    rng = np.random.default_rng(N * 7 + C * 3 + H + W + O + per_sample)
    x = rng.integers(-4, 5, size=(N, C, H, W)).astype(np.float32)
    wb = N if per_sample else 1
    w = rng.integers(-3, 4, size=(wb, O, C, 3, 3)).astype(np.float32)
    bias = rng.integers(-2, 3, size=(1, 1, H * W, O)).astype(np.float32)
    badd = bias.reshape(H, W, O).transpose(2, 0, 1)[None].astype(np.float64)
    w_ref = np.concatenate([oracle.weights_oihw_to_ref(w[b]) for b in range(wb)], axis=0)
    truth = np.concatenate([oracle.conv2d_direct_f64(x[b:b + 1], w[b if per_sample else 0], None, 1, 1) for b in range(N)], axis=0) + badd
    got = host(nz.conv2d_forward(dev(x), dev(w_ref), dev(bias), 3, 3, 1, 1, bias_strides=(O, 1), relu=False))
    assert np.array_equal(got.astype(np.float64), truth)


@pytest.mark.parametrize("N,C,H,W,O,k,pad,pix", PER_SAMPLE)
def test_conv2d_per_sample_weights_that_differ_between_images(nz, oracle, N, C, H, W, O, k, pad, pix):
    # the reference's Conv2d parameter holds one weight copy per sample (src/Model.cu:248-252); here every copy is
    # different, so a kernel that multiplied image b by another image's weights would be found out
    rng = np.random.default_rng(N + 3 * C + 5 * H + W + O + k)
    x = rng.integers(-4, 5, size=(N, C, H, W)).astype(np.float32)
    w = rng.integers(-3, 4, size=(N, O, C, k, k)).astype(np.float32)
    Ho, Wo = oracle.out_hw(H, W, k, k, 1, pad)
    if pix:
        bias = rng.integers(-2, 3, size=(1, 1, Ho * Wo, O)).astype(np.float32)
        strides, badd = (O, 1), bias.reshape(Ho, Wo, O).transpose(2, 0, 1)[None].astype(np.float64)
    else:
        bias = rng.integers(-2, 3, size=(O,)).astype(np.float32)
        strides, badd = (0, 1), bias.reshape(1, O, 1, 1).astype(np.float64)
    w_ref = np.concatenate([oracle.weights_oihw_to_ref(w[b]) for b in range(N)], axis=0)
    truth = np.concatenate([oracle.conv2d_direct_f64(x[b:b + 1], w[b], None, 1, pad) for b in range(N)], axis=0) + badd
    got = host(nz.conv2d_forward(dev(x), dev(w_ref), dev(bias), k, k, 1, pad, bias_strides=strides, relu=False))
    assert np.array_equal(got.astype(np.float64), truth)


def _conv_sweep_cases(seed, count):
    """Random geometries over every route: direct / streaming (few channels), implicit GEMM with 32- and 64-wide
    patches and both channel tiles, resident weights (single and double halo buffers), the column-matrix route
    (strides, 2x3 / 5x5 kernels), per-sample weights."""
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        k = int(rng.choice([1, 2, 3, 3, 3, 5]))
        k_w = 3 if k == 2 else k
        stride = int(rng.choice([1, 1, 1, 2]))
        pad = int(rng.integers(0, k_w))
        C = int(rng.choice([1, 3, 8, 17, 32, 50, 64, 70, 128]))
        O = int(rng.choice([1, 2, 5, 40, 64, 100, 128, 130]))
        H = int(rng.integers(max(k, 1), 20))
        W = int(rng.choice([int(rng.integers(max(k_w, 1), 40)), 64, 68, 72, 128, 132]))
        N = int(rng.integers(1, 4))
        wb = int(rng.choice([1, 1, 1, N]))
        Ho, Wo = (H + 2 * pad - k) // stride + 1, (W + 2 * pad - k_w) // stride + 1
        if Ho < 1 or Wo < 1 or N * O * Ho * Wo * C * k * k_w > 3e8:
            continue
        cases.append((N, C, H, W, O, k, k_w, stride, pad, wb))
    return cases


@pytest.mark.parametrize("N,C,H,W,O,k_h,k_w,stride,pad,w_batch", _conv_sweep_cases(20251, 64))
def test_conv2d_random_sweep_integers_bit_exact(nz, oracle, N, C, H, W, O, k_h, k_w, stride, pad, w_batch):
    rng = np.random.default_rng(N * 7 + C * 11 + H * 13 + W * 17 + O * 19 + k_h + stride + pad)
    x = rng.integers(-4, 5, size=(N, C, H, W)).astype(np.float32)
    bias = rng.integers(-2, 3, size=(O,)).astype(np.float32)
    ws = [rng.integers(-3, 4, size=(O, C, k_h, k_w)).astype(np.float32) for _ in range(w_batch)]
    w_ref = np.concatenate([oracle.weights_oihw_to_ref(w) for w in ws], axis=0)
    got = host(nz.conv2d_forward(dev(x), dev(w_ref), dev(bias), k_h, k_w, stride, pad, bias_strides=(0, 1), relu=True))
    for n in range(N):
        w = ws[n if w_batch > 1 else 0]
        truth = oracle.conv2d_direct_f64(x[n:n + 1], w, bias, stride, pad, relu=True)
        assert np.array_equal(got[n:n + 1].astype(np.float64), truth), (n,)


@pytest.mark.parametrize("N,C,H,W,O", [(2, 5, 10, 9, 6), (1, 128, 9, 64, 64), (1, 64, 8, 64, 128), (2, 64, 7, 64, 48), (1, 32, 8, 128, 64)])
def test_conv2d_per_pixel_bias_like_the_reference_parameter(nz, oracle, N, C, H, W, O):
    x = oracle.fill((N, C, H, W), 61, "normal", 0.0, 1.0)
    w = oracle.fill((O, C, 3, 3), 62, "normal", 0.0, 0.2)
    Ho, Wo = oracle.out_hw(H, W, 3, 3, 1, 1)
    bias_px = oracle.fill((1, 1, Ho * Wo, O), 63, "uniform", -0.5, 0.5)
    truth = oracle.conv2d_direct_f64(x, w, None, 1, 1) + bias_px.reshape(Ho, Wo, O).transpose(2, 0, 1)[None].astype(np.float64)
    got = host(nz.conv2d_forward(dev(x), dev(oracle.weights_oihw_to_ref(w)), dev(bias_px), 3, 3, 1, 1,
                                 bias_strides=(O, 1), relu=False))
    check_tolerance(oracle, got, truth, "per-pixel bias")
    ref = oracle.conv2d_graph(x, oracle.weights_oihw_to_ref(w), bias_px, 3, 3, 1, 1)
    assert np.max(np.abs(got - ref)) <= 1e-4


@pytest.mark.parametrize("N,C,H,W,O", [(2, 3, 40, 264, 1), (1, 2, 20, 8, 2), (2, 4, 17, 260, 2), (1, 1, 9, 12, 1)])
def test_stream_conv_with_the_reference_bias_layout_is_bit_exact(nz, oracle, N, C, H, W, O):
    """Few channels (the streaming kernel) with the bias parameter the reference's Model::Conv2d creates,
    [1, 1, H*W, O]: fetched as aligned runs of 4 pixels x O channels, or element by element when the bias
    pointer is not 16-byte aligned; both equal the im2col -> GEMM -> bias -> col2im -> ReLU graph bit for bit."""
    x = oracle.fill((N, C, H, W), 71, "uniform", 0.0, 1.0)
    w_ref = oracle.weights_oihw_to_ref(oracle.fill((O, C, 3, 3), 72, "normal", 0.0, 0.3))
    bias_px = oracle.fill((1, 1, H * W, O), 73, "uniform", -0.5, 0.5)
    want = np.maximum(oracle.conv2d_graph(x, w_ref, bias_px, 3, 3, 1, 1), 0)
    got = host(nz.conv2d_forward(dev(x), dev(w_ref), dev(bias_px), 3, 3, 1, 1, bias_strides=(O, 1), relu=True))
    assert np.array_equal(got, want)
    shifted = dev(np.concatenate([[0.0], bias_px.reshape(-1)]))[1:]              # 4-byte aligned only
    got2 = host(nz.conv2d_forward(dev(x), dev(w_ref), shifted, 3, 3, 1, 1, bias_strides=(O, 1), relu=True))
    assert np.array_equal(got2, want)


def test_config4a_conv_64_to_128_channels(nz, oracle):
    N, C, H, W, O = 16, 64, 128, 128, 128
    x = oracle.fill((N, C, H, W), 4, "normal", 0.0, 1.0)
    w = oracle.fill((O, C, 3, 3), 1004, "normal", 0.0, float(np.sqrt(2.0 / (C * 9))))
    bias = oracle.fill((O,), 2004, "uniform", -0.03, 0.03)
    got = nz.conv2d_forward(dev(x), dev(oracle.weights_oihw_to_ref(w)), dev(bias), 3, 3, 1, 1, bias_strides=(0, 1), relu=True)
    # two whole images against the fp64 direct convolution
    for b in (0, 11):
        truth = oracle.conv2d_direct_f64(x[b:b + 1], w, bias, 1, 1, relu=True)
        check_tolerance(oracle, host(got[b:b + 1]), truth, f"CA image {b}")
    # translation property at full size: shifting the batch order permutes the output
    perm = np.roll(np.arange(N), 3)
    got_p = nz.conv2d_forward(dev(x[perm]), dev(oracle.weights_oihw_to_ref(w)), dev(bias), 3, 3, 1, 1, bias_strides=(0, 1), relu=True)
    assert np.array_equal(host(got_p), host(got)[perm])


def test_config4b_conv_memory_bound_single_channel_out(nz, oracle):
    N, C, H, W, O = 10, 3, 1024, 1024, 1
    x = oracle.fill((N, C, H, W), 14, "uniform", 0.0, 1.0)
    w = oracle.fill((O, C, 3, 3), 1014, "normal", 0.0, float(np.sqrt(2.0 / 27)))
    bias = oracle.fill((O,), 2014, "uniform", -0.03, 0.03)
    got = host(nz.conv2d_forward(dev(x), dev(oracle.weights_oihw_to_ref(w)), dev(bias), 3, 3, 1, 1, bias_strides=(0, 1), relu=True))
    truth = oracle.conv2d_direct_f64(x, w, bias, 1, 1, relu=True)
    check_tolerance(oracle, got, truth, "CB")
