"""Parity of the HIP GEMM path (called through the C-ABI of include/nzhip.h) with the CPU
oracle.  Bar: bit-exact wherever arithmetic is exact (integer-valued operands, the
reference's literal vectors, identity products); otherwise the stated contract
max-rel <= 1e-3 and Frobenius-rel <= 1e-4 against an fp64 accumulation of the same
fp16-rounded inputs, where max-rel uses the RMS of the truth as the absolute floor
(|got-truth| / max(|truth|, rms(truth)))."""
import json
import os

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
    return mr, fr


def test_device_is_gfx950(nz):
    import ctypes as C
    cu, lds, name = C.c_int(0), C.c_size_t(0), C.create_string_buffer(64)
    nz.check(nz.load().nzhip_device_info(C.byref(cu), C.byref(lds), name, 64))
    assert name.value.decode().startswith("gfx950"), name.value
    assert cu.value >= 200 and lds.value >= 160 * 1024


def test_reference_literal_vectors(nz):
    with open(os.path.join(os.path.dirname(__file__), "golden", "matmul_broadcast.json")) as f:
        g = json.load(f)
    A = np.array(g["A"], np.float32).reshape(g["shapeA"])
    B = np.array(g["B"], np.float32).reshape(g["shapeB"])
    C = np.array(g["C"], np.float32).reshape(g["shapeC"])
    assert np.array_equal(host(nz.tensorcore_gemm(dev(A), dev(B))), C)


SHAPES = [(1, 1, 1), (3, 5, 2), (16, 16, 16), (17, 33, 15), (64, 100, 132), (130, 257, 67), (128, 32, 128),
          (256, 64, 256), (257, 31, 255), (300, 40, 520), (1000, 777, 513), (1, 4096, 64), (8, 8, 1024)]


@pytest.mark.parametrize("M,K,N", SHAPES)
@pytest.mark.parametrize("a_trans,b_trans", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("tile", [64, 128, 256, 16, 18, 12, 316, 318, 312])  # fused kernels with that tile; 16 / 18 / 12 = two-pass fp16 route variants (16x16x32 MFMAs), 3xx = the same with 32x32x16
def test_integer_operands_are_bit_exact(nz, M, K, N, a_trans, b_trans, tile):
    rng = np.random.default_rng(M * 7919 + K * 31 + N)
    A = rng.integers(-8, 9, size=(M, K)).astype(np.float32)
    B = rng.integers(-8, 9, size=(K, N)).astype(np.float32)
    expect = (A.astype(np.int64) @ B.astype(np.int64)).astype(np.float32)
    Ad = dev(A.T if a_trans else A)
    Bd = dev(B.T if b_trans else B)
    got = host(nz.gemm(Ad, Bd, a_trans=a_trans, b_trans=b_trans, force_tile=tile))
    assert np.array_equal(got, expect)


SKINNY = [(1, 1, 1), (1, 4096, 64), (1, 777, 513), (3, 300, 1000), (8, 64, 260), (5, 1000, 7), (1000, 77, 3),
          (300, 40, 1), (2049, 130, 8), (7, 9, 4100), (1, 5, 3),
          # long and wide enough for the kernel that keeps the whole contraction in one workgroup (when the long
          # operand has its long extent contiguous): K a multiple of its row step and not, one and two skinny rows
          (1, 4096, 4096), (2, 1500, 2064), (2048, 1100, 2), (4096, 1024, 1)]


@pytest.mark.parametrize("M,K,N", SKINNY)
@pytest.mark.parametrize("a_trans,b_trans", [(False, False), (False, True), (True, False), (True, True)])
def test_skinny_products_are_bit_exact_on_integers(nz, M, K, N, a_trans, b_trans):
    # min(M, N) <= 8: the bandwidth-bound streaming kernels (up to 2 rows / 3 columns, or K < 512) or the MFMA
    # kernel with a split contraction; bias and ReLU ride along
    rng = np.random.default_rng(M * 31 + K * 7 + N)
    A = rng.integers(-8, 9, size=(M, K)).astype(np.float32)
    B = rng.integers(-8, 9, size=(K, N)).astype(np.float32)
    bias = rng.integers(-50, 51, size=(M, N)).astype(np.float32)
    expect = np.maximum((A.astype(np.int64) @ B.astype(np.int64)).astype(np.float32) + bias, 0)
    got = host(nz.gemm(dev(A.T if a_trans else A), dev(B.T if b_trans else B), a_trans=a_trans, b_trans=b_trans,
                       bias=dev(bias), bias_strides=(N, 1), relu=True))
    assert np.array_equal(got, expect)


def test_skinny_split_contraction_back_to_back(nz):
    # the streaming kernel's blocks leave partial sums in a pooled workspace that a second kernel adds: calls of
    # different shapes, queued without a wait between them on two streams, must not see each other's partials
    import torch
    shapes = [(1, 4096, 4096), (2, 3000, 700), (1, 4096, 4096), (1, 777, 513), (2, 1024, 260)]
    side = torch.cuda.Stream()
    todo = []
    for rep in range(3):
        for i, (M, K, N) in enumerate(shapes):
            rng = np.random.default_rng(rep * 100 + i)
            A = rng.integers(-8, 9, size=(M, K)).astype(np.float32)
            B = rng.integers(-8, 9, size=(K, N)).astype(np.float32)
            todo.append((dev(A), dev(B), (A.astype(np.int64) @ B.astype(np.int64)).astype(np.float32)))
    torch.cuda.synchronize()
    outs = []
    for j, (Ad, Bd, _) in enumerate(todo):
        if j % 2:
            with torch.cuda.stream(side):
                outs.append(nz.gemm(Ad, Bd, stream=side))
        else:
            outs.append(nz.gemm(Ad, Bd))
    torch.cuda.synchronize()
    for (_, _, expect), got in zip(todo, outs):
        assert np.array_equal(host(got), expect)


SPLITK = [(130, 9000, 70), (576, 16384, 128), (64, 4096, 64), (33, 20001, 300), (128, 8192, 129),
          (10, 70000, 16), (16, 33000, 10)]       # a handful of outputs, hundreds of chunks: one wave per output adds them


@pytest.mark.parametrize("M,K,N", SPLITK)
@pytest.mark.parametrize("a_trans,b_trans", [(False, False), (False, True), (True, False), (True, True)])
def test_long_contractions_with_few_tiles_are_bit_exact_on_integers(nz, M, K, N, a_trans, b_trans):
    # few output tiles and a long contraction: it is cut into chunks that are added in order;
    # a full [M,N] bias and ReLU are applied once, after the last chunk
    rng = np.random.default_rng(M * 13 + K + N * 5)
    A = rng.integers(-4, 5, size=(M, K)).astype(np.float32)
    B = rng.integers(-4, 5, size=(K, N)).astype(np.float32)
    bias = rng.integers(-50, 51, size=(M, N)).astype(np.float32)
    expect = np.maximum((A.astype(np.int64) @ B.astype(np.int64)).astype(np.float32) + bias, 0)
    got = host(nz.gemm(dev(A.T if a_trans else A), dev(B.T if b_trans else B), a_trans=a_trans, b_trans=b_trans,
                       bias=dev(bias), bias_strides=(N, 1), relu=True))
    assert np.array_equal(got, expect)


@pytest.mark.parametrize("M,K,N", [(300, 1000, 260), (130, 9000, 70), (999, 777, 513), (1024, 2048, 1024), (64, 64, 64)])
@pytest.mark.parametrize("force", [0, 64, 128, 256, 18, 12])
def test_bias_may_alias_the_output(nz, M, K, N, force):
    # "C += A B": the bias operand is C itself, element for element. Every route reads bias(m, n) in the
    # thread that writes C(m, n), also behind a split contraction or padded operand copies.
    rng = np.random.default_rng(M + 3 * K + 5 * N + force)
    A = rng.integers(-4, 5, size=(M, K)).astype(np.float32)
    B = rng.integers(-4, 5, size=(K, N)).astype(np.float32)
    C0 = rng.integers(-100, 101, size=(M, N)).astype(np.float32)
    expect = (A.astype(np.int64) @ B.astype(np.int64)).astype(np.float32) + C0
    Cd = dev(C0)
    nz.gemm(dev(A), dev(B), bias=Cd, bias_strides=(N, 1), out=Cd, force_tile=force)
    assert np.array_equal(host(Cd), expect)


COOP = [(4096, 2048, 4096), (8192, 1024, 4096), (4096, 1024, 8192), (8192, 2048, 8192)]


@pytest.mark.parametrize("M,K,N", COOP)
@pytest.mark.parametrize("a_trans,b_trans", [(False, False), (False, True), (True, False), (True, True)])
def test_single_kernel_route_is_bit_exact_on_integers(nz, M, K, N, a_trans, b_trans):
    # the route for very large products (rounding done inside the k loops of the GEMM, stage counters between
    # workgroups): one wave of tiles with two panels; two waves that share B, or A; four waves in boustrophedon
    # order. Bias matrix and ReLU ride along; no wait may have run out.
    import ctypes as C
    import torch
    gen = torch.Generator(device="cuda").manual_seed(M + 3 * K + 7 * N + 2 * a_trans + b_trans)
    A = torch.randint(-4, 5, (K, M) if a_trans else (M, K), generator=gen, device="cuda").float()
    B = torch.randint(-4, 5, (N, K) if b_trans else (K, N), generator=gen, device="cuda").float()
    bias = torch.randint(-50, 51, (M, N), generator=gen, device="cuda").float()
    expect = torch.relu(((A.T if a_trans else A).double() @ (B.T if b_trans else B).double()).float() + bias)   # |sums| < 2^24: exact
    got = nz.gemm(A, B, a_trans=a_trans, b_trans=b_trans, bias=bias, bias_strides=(N, 1), relu=True, force_tile=28)
    assert torch.equal(got, expect)
    again = nz.gemm(A, B, a_trans=a_trans, b_trans=b_trans, bias=bias, bias_strides=(N, 1), relu=True)      # default route: the same one
    assert torch.equal(again, expect)
    n = C.c_uint(123)
    nz.check(nz.load().nzhip_gemm_coop_timeouts(C.byref(n)))
    assert n.value == 0


def test_single_kernel_route_bias_forms(nz):
    # no bias; a per-column vector (the Linear layer's form); a per-row vector; all against the two-kernel route,
    # which must give the same bits (same tiles, same k order)
    import torch
    M, K, N = 4096, 2048, 4096
    gen = torch.Generator(device="cuda").manual_seed(99)
    A = (torch.rand((M, K), generator=gen, device="cuda") - 0.5)
    B = (torch.rand((K, N), generator=gen, device="cuda") - 0.5)
    col = torch.rand((N,), generator=gen, device="cuda") - 0.5
    row = torch.rand((M,), generator=gen, device="cuda") - 0.5
    for kw in (dict(), dict(bias=col, bias_strides=(0, 1), relu=True), dict(bias=row, bias_strides=(1, 0))):
        one = nz.gemm(A, B, force_tile=28, **kw)
        two = nz.gemm(A, B, force_tile=18, **kw)
        assert torch.equal(one, two), kw.keys()


def test_single_kernel_route_rejects_other_shapes(nz):
    import torch
    A, B = torch.zeros((4096, 1000), device="cuda"), torch.zeros((1000, 4096), device="cuda")
    with pytest.raises(nz.NzHipError) as e:
        nz.gemm(A, B, force_tile=28)
    assert e.value.status == -3


def test_single_kernel_route_reports_waits_that_ran_out(nz):
    # A bounded wait that runs out leaves a product that may be wrong. No kernel is made to misbehave here: the
    # device-side count is raised from the host after a (correct) product, and the runtime must then say so at
    # the first blocking call that has drained the product's stream, once, and stop taking the route.
    import ctypes as C
    import torch
    lib = nz.load()
    M, K, N = 4096, 2048, 4096
    rng = np.random.default_rng(3)
    A = dev(rng.integers(-4, 5, size=(M, K)).astype(np.float32))
    B = dev(rng.integers(-4, 5, size=(K, N)).astype(np.float32))
    want = nz.gemm(A, B, force_tile=18)
    torch.cuda.synchronize()
    nz.check(lib.nzhip_gemm_coop_reset(0))
    rt = torch.cuda.ExternalStream(lib.nzhip_default_stream())
    try:
        got = nz.gemm(A, B, force_tile=28, stream=rt)          # on the runtime's stream: nzhip_sync_ptr covers it
        nz.check(lib.nzhip_sync_ptr(None))                         # nothing ran out: no complaint
        assert torch.equal(got, want)
        got = nz.gemm(A, B, force_tile=28, stream=rt)
        nz.check(lib.nzhip_gemm_coop_reset(2))                     # "two waits ran out"
        with pytest.raises(nz.NzHipError) as e:
            nz.check(lib.nzhip_sync_ptr(None))
        assert e.value.status == -5 and "2 bounded waits" in str(e.value)
        nz.check(lib.nzhip_sync_ptr(None))                         # reported once
        with pytest.raises(nz.NzHipError) as e:                    # the route is off now ...
            nz.gemm(A, B, force_tile=28)
        assert e.value.status == -3
        assert torch.equal(nz.gemm(A, B), want)                    # ... and the default route still multiplies
        # a product on another stream is only looked at once the whole device has been drained
        nz.check(lib.nzhip_gemm_coop_reset(0))
        got = nz.gemm(A, B, force_tile=28)                         # torch's current stream
        nz.check(lib.nzhip_gemm_coop_reset(1))
        nz.check(lib.nzhip_sync_ptr(None))
        with pytest.raises(nz.NzHipError) as e:
            nz.check(lib.nzhip_sync_all())
        assert e.value.status == -5
    finally:
        nz.check(lib.nzhip_gemm_coop_reset(0))
    torch.cuda.synchronize()
    assert torch.equal(nz.gemm(A, B, force_tile=28), want)


def test_single_kernel_route_writes_nan_when_a_wait_runs_out(nz):
    # The waits are made to run out from the host: producers keep their arrivals to themselves and a wait gives
    # up after one poll. Every wave still runs to the end of the kernel; the product must then be NaN all over
    # (never a plausible wrong number), the runtime must say so at the next blocking call, and the route must
    # work again once the hook is off.
    import torch
    lib = nz.load()
    M, K, N = 4096, 2048, 4096
    gen = torch.Generator(device="cuda").manual_seed(17)
    A = torch.randint(-4, 5, (M, K), generator=gen, device="cuda").float()
    B = torch.randint(-4, 5, (K, N), generator=gen, device="cuda").float()
    want = nz.gemm(A, B, force_tile=18)
    torch.cuda.synchronize()
    nz.check(lib.nzhip_gemm_coop_reset(0))
    try:
        nz.check(lib.nzhip_gemm_coop_test_mode(1, 1))
        got = torch.zeros((M, N), device="cuda")
        nz.gemm(A, B, out=got, force_tile=28)
        torch.cuda.synchronize()
        assert bool(torch.isnan(got).all())
        with pytest.raises(nz.NzHipError) as e:
            nz.check(lib.nzhip_sync_all())
        assert e.value.status == -5 and "NaN" in str(e.value)
    finally:
        nz.check(lib.nzhip_gemm_coop_test_mode(0, 0))
        nz.check(lib.nzhip_gemm_coop_reset(0))
    assert torch.equal(nz.gemm(A, B, force_tile=28), want)


@pytest.mark.parametrize("b_trans", [False, True])
def test_single_kernel_route_equals_two_kernel_route_at_8192_cubed(nz, b_trans):
    # the benchmarked shape in full (four waves of workgroups, eight panels), float data: both routes run the
    # same tiles in the same k order, so every one of the 2^26 outputs must have the same bits; and a sample of
    # rows agrees with fp64 accumulation of the rounded operands
    import ctypes as C
    import torch
    n = 8192
    gen = torch.Generator(device="cuda").manual_seed(8192 + b_trans)
    A = torch.randn((n, n), generator=gen, device="cuda") / n ** 0.5
    B = torch.randn((n, n), generator=gen, device="cuda") / n ** 0.5
    one = nz.gemm(A, B, b_trans=b_trans, force_tile=28)
    two = nz.gemm(A, B, b_trans=b_trans, force_tile=18)
    assert torch.equal(one, two)
    rows = torch.arange(0, n, 257, device="cuda")
    Ah, Bh = A[rows].half().double(), B.half().double()
    truth = Ah @ (Bh.T if b_trans else Bh)
    err = (one[rows].double() - truth).abs().max() / truth.pow(2).mean().sqrt()
    assert float(err) <= 1e-3
    cnt = C.c_uint(123)
    nz.check(nz.load().nzhip_gemm_coop_timeouts(C.byref(cnt)))
    assert cnt.value == 0


def _route_sweep_cases():
    # seeded shapes aimed at the boundaries of the route choice: skinny extents 1..9 on either side,
    # long contractions with few tiles (split or not, vectorisable or not), mid-size and ragged shapes,
    # and two shapes big enough for the two-pass route under the default rule
    rng = np.random.default_rng(20240607)
    cases = []
    for _ in range(10):
        cases.append((int(rng.integers(1, 10)), int(rng.integers(400, 3000)), int(rng.integers(100, 1500))))
        cases.append((int(rng.integers(100, 1500)), int(rng.integers(400, 3000)), int(rng.integers(1, 10))))
    for _ in range(10):
        cases.append((int(rng.integers(10, 400)), int(rng.integers(500, 6000)), int(rng.integers(10, 400))))
        cases.append((4 * int(rng.integers(3, 100)), 4 * int(rng.integers(128, 1500)), 4 * int(rng.integers(3, 100))))
    for _ in range(6):
        cases.append((int(rng.integers(200, 900)), int(rng.integers(30, 700)), int(rng.integers(200, 900))))
    cases += [(1800, 800, 1804), (1024, 1024, 1024), (512, 768, 2048), (1792, 1024, 1792)]
    return cases


@pytest.mark.parametrize("M,K,N", _route_sweep_cases())
def test_default_route_is_bit_exact_on_integers(nz, M, K, N):
    # no forced kernel: whatever nzhip_gemm picks for the shape must give the exact integer product
    rng = np.random.default_rng(M * 1009 + K * 17 + N)
    a_trans, b_trans = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    A = rng.integers(-4, 5, size=(M, K)).astype(np.float32)
    B = rng.integers(-4, 5, size=(K, N)).astype(np.float32)
    bias = rng.integers(-50, 51, size=(N,)).astype(np.float32)
    # float64 BLAS is exact here: |sum| <= 16 K < 2^53
    expect = np.maximum((A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32) + bias[None, :], 0)
    got = host(nz.gemm(dev(np.ascontiguousarray(A.T) if a_trans else A), dev(np.ascontiguousarray(B.T) if b_trans else B),
                       a_trans=a_trans, b_trans=b_trans, bias=dev(bias), bias_strides=(0, 1), relu=True))
    assert np.array_equal(got, expect)



def test_skinny_batched_linear_single_sample(nz, oracle):
    # one sample through Model::Linear: W[1,1,OUT,IN] x[1,1,IN,1]
    OUT, IN = 1000, 515
    W = oracle.fill((1, 1, OUT, IN), 71, "uniform", -0.1, 0.1)
    x = oracle.fill((1, 1, IN, 1), 72, "normal", 0.0, 1.0)
    got = host(nz.tensorcore_gemm(dev(W), dev(x))).reshape(OUT)
    truth = oracle.gemm_f64(W.reshape(OUT, IN), x.reshape(IN, 1)).reshape(OUT)
    check_tolerance(oracle, got, truth, "single-sample linear")
    # batched GEMVs that cannot be collapsed (both operands batched): [3,2,1,64] x [3,2,64,300]
    A = oracle.fill((3, 2, 1, 64), 73, "uniform", -1.0, 1.0)
    Bm = oracle.fill((3, 2, 64, 300), 74, "uniform", -1.0, 1.0)
    got = host(nz.tensorcore_gemm(dev(A), dev(Bm)))
    ref = oracle.tensorcore_gemm(A, Bm)
    assert np.max(np.abs(got - ref)) <= 1e-4


@pytest.mark.parametrize("M,K,N", [(1000, 777, 513), (700, 701, 333), (999, 1001, 1003), (516, 1030, 520)])
@pytest.mark.parametrize("a_trans,b_trans", [(False, False), (False, True), (True, False), (True, True)])
def test_operands_without_16_byte_rows_are_bit_exact_on_integers(nz, M, K, N, a_trans, b_trans):
    # products big enough for it are computed from zero-padded copies of the operands whose rows do not allow
    # 16-byte loads; rows are embedded in NaN-filled storage with a leading dimension of their own and an odd base
    # offset, so a read past a row's end or a missing zero in the padding poisons the result
    import ctypes as C
    import torch
    rng = np.random.default_rng(M + 3 * K + 7 * N)
    A = rng.integers(-8, 9, size=(M, K)).astype(np.float32)
    B = rng.integers(-8, 9, size=(K, N)).astype(np.float32)
    bias = rng.integers(-50, 51, size=(M, N)).astype(np.float32)
    expect = np.maximum((A.astype(np.int64) @ B.astype(np.int64)).astype(np.float32) + bias, 0)

    def embed(X, ld, off):
        rows, cols = X.shape
        buf = torch.full((rows * ld + off + 8,), float("nan"), device="cuda")
        view = buf[off:off + rows * ld].view(rows, ld)
        view[:, :cols] = torch.from_numpy(X).cuda()
        return buf, view.data_ptr()

    As = A.T.copy() if a_trans else A
    Bs = B.T.copy() if b_trans else B
    lda, ldb, ldc = As.shape[1] + 2, Bs.shape[1] + 1, N + 3
    bufA, pa = embed(As, lda, 1)
    bufB, pb = embed(Bs, ldb, 3)
    out = torch.full((M * ldc + 1,), float("nan"), device="cuda")
    bd = dev(bias)
    d = nz.GemmDesc()
    d.A, d.B, d.C = pa, pb, out.data_ptr() + 4
    d.M, d.N, d.K = M, N, K
    d.lda, d.ldb, d.ldc = lda, ldb, ldc
    d.a_layout = nz.LAYOUT_TRANS if a_trans else nz.LAYOUT_ROW
    d.b_layout = nz.LAYOUT_TRANS if b_trans else nz.LAYOUT_ROW
    d.batch_n = d.batch_c = 1
    d.bias = bd.data_ptr()
    d.bias_stride_row, d.bias_stride_col = N, 1
    d.activation = nz.ACT_RELU
    nz.check(nz.load().nzhip_gemm(C.byref(d), None))
    torch.cuda.synchronize()
    got = out[1:].view(M, ldc).cpu().numpy()
    assert np.array_equal(got[:, :N], expect)
    assert np.all(np.isnan(got[:, N:]))                            # nothing written between the rows of C


def _embedded_cases():
    rng = np.random.default_rng(777)
    cases = []
    for i in range(96):
        big = i % 3 == 0
        M = int(rng.integers(1, 1200 if big else 200))
        N = int(rng.integers(1, 1200 if big else 200))
        K = int(rng.integers(1, 2500 if big else 400))
        cases.append((M, K, N, bool(rng.integers(2)), bool(rng.integers(2)), [int(v) for v in rng.integers(0, 6, size=3)],
                      [int(v) for v in rng.integers(0, 4, size=3)], int(rng.integers(4)), 1000 + i))
    return cases


@pytest.mark.parametrize("M,K,N,a_trans,b_trans,slack,offset,bias_form,seed", _embedded_cases())
def test_embedded_operands_random_sweep(nz, M, K, N, a_trans, b_trans, slack, offset, bias_form, seed):
    # random shapes, layouts, leading dimensions and base offsets through the default route choice (streaming,
    # thin, split, 64 / 128 tiles, padded copies): exact on integers, nothing read or written outside the rows
    import ctypes as C
    import torch
    rng = np.random.default_rng(seed)
    A = rng.integers(-4, 5, size=(M, K)).astype(np.float32)
    B = rng.integers(-4, 5, size=(K, N)).astype(np.float32)
    expect = (A.astype(np.int64) @ B.astype(np.int64)).astype(np.float32)
    bias = None
    if bias_form == 1:                                              # one value per column
        bias = rng.integers(-50, 51, size=(N,)).astype(np.float32)
        expect = expect + bias[None, :]
        strides = (0, 1)
    elif bias_form == 2:                                            # one value per row
        bias = rng.integers(-50, 51, size=(M,)).astype(np.float32)
        expect = expect + bias[:, None]
        strides = (1, 0)
    elif bias_form == 3:                                            # a full matrix, and ReLU
        bias = rng.integers(-50, 51, size=(M, N)).astype(np.float32)
        expect = np.maximum(expect + bias, 0)
        strides = (N, 1)

    def embed(X, ld, off):
        rows, cols = X.shape
        buf = torch.full((rows * ld + off + 8,), float("nan"), device="cuda")
        buf[off:off + rows * ld].view(rows, ld)[:, :cols] = torch.from_numpy(X).cuda()
        return buf, buf.data_ptr() + 4 * off

    As = A.T.copy() if a_trans else A
    Bs = B.T.copy() if b_trans else B
    lda, ldb, ldc = As.shape[1] + slack[0], Bs.shape[1] + slack[1], N + slack[2]
    bufA, pa = embed(As, lda, offset[0])
    bufB, pb = embed(Bs, ldb, offset[1])
    out = torch.full((M * ldc + offset[2] + 8,), float("nan"), device="cuda")
    d = nz.GemmDesc()
    d.A, d.B, d.C = pa, pb, out.data_ptr() + 4 * offset[2]
    d.M, d.N, d.K = M, N, K
    d.lda, d.ldb, d.ldc = lda, ldb, ldc
    d.a_layout = nz.LAYOUT_TRANS if a_trans else nz.LAYOUT_ROW
    d.b_layout = nz.LAYOUT_TRANS if b_trans else nz.LAYOUT_ROW
    d.batch_n = d.batch_c = 1
    if bias is not None:
        bd = dev(bias)
        d.bias = bd.data_ptr()
        d.bias_stride_row, d.bias_stride_col = strides
        d.activation = nz.ACT_RELU if bias_form == 3 else nz.ACT_NONE
    nz.check(nz.load().nzhip_gemm(C.byref(d), None))
    torch.cuda.synchronize()
    flat = out.cpu().numpy()
    got = flat[offset[2]:offset[2] + M * ldc].reshape(M, ldc)
    assert np.array_equal(got[:, :N], expect)
    assert np.all(np.isnan(got[:, N:])) and np.all(np.isnan(flat[:offset[2]])) and np.all(np.isnan(flat[offset[2] + M * ldc:]))


def test_unaligned_base_pointers_take_the_scalar_path(nz):
    import torch
    rng = np.random.default_rng(5)
    M, K, N = 70, 52, 36
    A = rng.integers(-8, 9, size=(M, K)).astype(np.float32)
    B = rng.integers(-8, 9, size=(K, N)).astype(np.float32)
    bufA = torch.zeros(M * K + 1, device="cuda")
    bufB = torch.zeros(K * N + 3, device="cuda")
    Ad = bufA[1:].view(M, K)
    Bd = bufB[3:].view(K, N)
    Ad.copy_(torch.from_numpy(A))
    Bd.copy_(torch.from_numpy(B))
    assert Ad.data_ptr() % 16 != 0 and Bd.data_ptr() % 16 != 0
    got = host(nz.gemm(Ad, Bd))
    assert np.array_equal(got, (A.astype(np.int64) @ B.astype(np.int64)).astype(np.float32))


def test_identity_gives_fp16_rounding_including_special_values(nz, oracle):
    n = 96
    X = oracle.fill((n, n), 11, "uniform", -4.0, 4.0)
    X[0, :12] = [65504.0, 65519.0, 65520.0, 1e6, -1e6, 2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -25, 6.0e-8, -2.0 ** -14,
                 3.0e-5, 1.0 + 2.0 ** -11]
    got = host(nz.gemm(dev(np.eye(n, dtype=np.float32)), dev(X)))
    expect = oracle.round_f16(X)                       # I * X = f16(X): zeros elsewhere add exactly
    # 0 * inf = NaN in the columns that hold an infinity after rounding; compare those apart
    inf_cols = np.isinf(expect).any(axis=0)
    assert np.array_equal(got[:, ~inf_cols].view(np.uint32) & 0x7FFFFFFF, expect[:, ~inf_cols].view(np.uint32) & 0x7FFFFFFF)
    assert np.all(np.isnan(got[1:, inf_cols])) and np.all(np.isinf(got[0, inf_cols]))
    # subnormal halfs survive the MFMA (no flush to zero)
    assert got[0, 5] == 2.0 ** -24 and got[0, 6] == 0.0 and got[0, 7] == 2.0 ** -24
    got_r = host(nz.gemm(dev(X), dev(np.eye(n, dtype=np.float32))))
    assert np.array_equal(got_r[1:], expect[1:])


def test_config1_gemm_256_uniform(nz, oracle):
    A = oracle.fill((256, 256), 0, "uniform", -1.0, 1.0)
    B = oracle.fill((256, 256), 1000, "uniform", -1.0, 1.0)
    truth = oracle.gemm_f64(A, B)
    for tile in (64, 128, 256, 16):
        got = host(nz.gemm(dev(A), dev(B), force_tile=tile))
        check_tolerance(oracle, got, truth, f"G1 tile {tile}")
        # and against the fp32 sequential oracle: same rounding, only the sum order differs
        ref32 = oracle.gemm(A, B)
        assert np.max(np.abs(got - ref32)) <= 256 * 2.0 ** -23 * np.max(np.abs(truth))


def test_config3_ragged_and_gemv(nz, oracle):
    A = oracle.fill((1000, 777), 3, "uniform", -1.0, 1.0)
    B = oracle.fill((777, 513), 1003, "uniform", -1.0, 1.0)
    check_tolerance(oracle, host(nz.gemm(dev(A), dev(B))), oracle.gemm_f64(A, B), "R1")
    a = oracle.fill((1, 4096), 4, "uniform", -1.0, 1.0)
    Bm = oracle.fill((4096, 4096), 1004, "uniform", -1.0, 1.0)
    check_tolerance(oracle, host(nz.gemm(dev(a), dev(Bm))), oracle.gemm_f64(a, Bm), "R2")


def test_config2_linear_bias_relu(nz, oracle):
    Nb, IN, OUT = 4096, 1024, 4096
    X = oracle.fill((Nb, IN), 2, "normal", 0.0, 1.0)
    bound = float(np.sqrt(6.0 / IN))
    Wt = oracle.fill((OUT, IN), 1002, "uniform", -bound, bound)       # reference storage [1,1,OUT,IN]
    bias = oracle.fill((OUT,), 2002, "uniform", -0.03, 0.03)
    expect32 = oracle.linear_graph(X, Wt, bias, relu=True)
    truth = oracle.gemm_f64(X, Wt, trans_b=True) + bias.astype(np.float64)[None, :]
    truth = np.maximum(truth, 0.0)
    # (1) fused form: Y[Nb,OUT] = relu(X * Wt^T + bias)
    got = host(nz.gemm(dev(X), dev(Wt), b_trans=True, bias=dev(bias), bias_strides=(0, 1), relu=True))
    check_tolerance(oracle, got, truth, "L fused")
    assert np.max(np.abs(got - expect32)) <= 1e-3
    assert np.array_equal(got == 0.0, np.maximum(got, 0) == 0.0) and got.min() >= 0.0
    # (2) config form W[K,N] row-major
    W = np.ascontiguousarray(Wt.T)
    got2 = host(nz.gemm(dev(X), dev(W), bias=dev(bias), bias_strides=(0, 1), relu=True))
    check_tolerance(oracle, got2, truth, "L config form")
    # (3) the graph exactly as Model::Linear builds it: W[1,1,OUT,IN] x[N,1,IN,1] -> [N,1,OUT,1]
    y = nz.tensorcore_gemm(dev(Wt.reshape(1, 1, OUT, IN)), dev(X.reshape(Nb, 1, IN, 1)))
    y = nz.relu(nz.add_broadcast(y, dev(bias.reshape(1, 1, OUT, 1))))
    check_tolerance(oracle, host(y).reshape(Nb, OUT), truth, "L graph")


@pytest.mark.parametrize("sa,sb", [((2, 1, 2, 3), (1, 3, 3, 2)), ((3, 2, 5, 7), (3, 2, 7, 4)), ((1, 1, 9, 6), (4, 1, 6, 1)),
                                    ((2, 3, 4, 5), (1, 1, 5, 6)), ((1, 3, 4, 5), (2, 1, 5, 6)), ((5, 1, 1, 40), (1, 1, 40, 24)),
                                    ((4, 2, 130, 70), (1, 2, 70, 260)), ((1, 1, 33, 20), (3, 4, 20, 1))])
def test_batched_broadcast_matches_oracle(nz, oracle, sa, sb):
    rng = np.random.default_rng(sum(sa) * 3 + sum(sb))
    A = rng.integers(-6, 7, size=sa).astype(np.float32)
    B = rng.integers(-6, 7, size=sb).astype(np.float32)
    assert np.array_equal(host(nz.tensorcore_gemm(dev(A), dev(B))), oracle.tensorcore_gemm(A, B))


@pytest.mark.parametrize("sa,sb", [((255, 257, 3, 5), (255, 257, 5, 2)),       # 65 535 members, skinny kernels
                                   ((255, 257, 9, 16), (1, 257, 16, 9)),       # 65 535 members, MFMA kernel, A-side n broadcast
                                   ((300, 300, 2, 3), (300, 1, 3, 2))])        # 90 000 members: split into several launches
def test_largest_batches(nz, sa, sb):
    rng = np.random.default_rng(sa[0] + sa[2])
    A = rng.integers(-6, 7, size=sa).astype(np.float32)
    B = rng.integers(-6, 7, size=sb).astype(np.float32)
    expect = np.matmul(A.astype(np.float64), B.astype(np.float64)).astype(np.float32)   # broadcasts n and c like the reference
    assert np.array_equal(host(nz.tensorcore_gemm(dev(A), dev(B))), expect)


@pytest.mark.parametrize("sa,sb", [((4, 1, 100, 1500), (1, 1, 1500, 130)),       # 4 members x 2 tiles, B shared
                                   ((3, 1, 130, 1100), (3, 1, 1100, 70)),        # both batched over n
                                   ((2, 1, 257, 4608), (1, 1, 4608, 250))])      # the column-matrix conv shape, small images
def test_batched_products_with_few_tiles_split_the_contraction(nz, sa, sb):
    """Products batched over n whose tiles leave most CUs idle run their contraction in chunks (a
    workspace of partial sums per member, added in a fixed order): exact on integers."""
    rng = np.random.default_rng(sa[2] + sb[3])
    A = rng.integers(-4, 5, size=sa).astype(np.float32)
    B = rng.integers(-4, 5, size=sb).astype(np.float32)
    expect = np.matmul(A.astype(np.float64), B.astype(np.float64)).astype(np.float32)
    assert np.array_equal(host(nz.tensorcore_gemm(dev(A), dev(B))), expect)


@pytest.mark.parametrize("M,K,N", [(16, 10, 5000), (5000, 16, 10), (3, 32, 4099), (2500, 1, 16), (9, 7, 2048), (2049, 31, 13)])
@pytest.mark.parametrize("a_trans,b_trans", [(False, False), (False, True), (True, False), (True, True)])
def test_thin_products_short_contraction_one_narrow_extent(nz, oracle, M, K, N, a_trans, b_trans):
    """K <= 32, one extent <= 16 and the other long (Linear-layer gradients with a huge fan-in): the streaming
    kernel, exact on integers with bias and ReLU, and bit-identical to the k-ascending oracle on float data."""
    rng = np.random.default_rng(M + 3 * K + 7 * N)
    A = rng.integers(-4, 5, size=(K, M) if a_trans else (M, K)).astype(np.float32)
    B = rng.integers(-4, 5, size=(N, K) if b_trans else (K, N)).astype(np.float32)
    bias = rng.integers(-5, 6, size=(M, N)).astype(np.float32)
    P = (A.T if a_trans else A).astype(np.int64) @ (B.T if b_trans else B).astype(np.int64)
    got = host(nz.gemm(dev(A), dev(B), a_trans=a_trans, b_trans=b_trans, bias=dev(bias), bias_strides=(N, 1), relu=True))
    assert np.array_equal(got, np.maximum(P + bias, 0).astype(np.float32))
    Af = rng.standard_normal(A.shape).astype(np.float32)
    Bf = rng.standard_normal(B.shape).astype(np.float32)
    want = oracle.gemm(np.ascontiguousarray(Af.T if a_trans else Af), np.ascontiguousarray(Bf.T if b_trans else Bf))
    assert np.array_equal(host(nz.gemm(dev(Af), dev(Bf), a_trans=a_trans, b_trans=b_trans)), want)
    # accumulate in place: the bias operand is the output itself
    out = dev(bias)
    nz.gemm(dev(A), dev(B), a_trans=a_trans, b_trans=b_trans, bias=out, bias_strides=(N, 1), out=out)
    assert np.array_equal(host(out), (P + bias).astype(np.float32))


def test_bias_forms_and_relu_special_values(nz, oracle):
    M, K, N = 40, 24, 52
    rng = np.random.default_rng(1)
    A = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
    B = rng.integers(-3, 4, size=(K, N)).astype(np.float32)
    P = (A.astype(np.int64) @ B.astype(np.int64)).astype(np.float32)
    row = rng.integers(-5, 6, size=(M,)).astype(np.float32)
    col = rng.integers(-5, 6, size=(N,)).astype(np.float32)
    full = rng.integers(-5, 6, size=(M, N)).astype(np.float32)
    assert np.array_equal(host(nz.gemm(dev(A), dev(B), bias=dev(row), bias_strides=(1, 0))), P + row[:, None])
    assert np.array_equal(host(nz.gemm(dev(A), dev(B), bias=dev(col), bias_strides=(0, 1))), P + col[None, :])
    assert np.array_equal(host(nz.gemm(dev(A), dev(B), bias=dev(full), bias_strides=(N, 1), relu=True)),
                          np.maximum(P + full, 0))
    # ReLU: NaN -> 0, -0 -> +0  (x > 0 ? x : 0, src/OperationKernels.cu:230-235)
    nanbias = np.zeros((M, N), np.float32)
    nanbias[0, 0] = np.nan
    nanbias[0, 1] = -np.inf
    out = host(nz.gemm(dev(np.zeros_like(A)), dev(B), bias=dev(nanbias), bias_strides=(N, 1), relu=True))
    assert out[0, 0] == 0.0 and out[0, 1] == 0.0 and not np.signbit(out).any()
    v = np.array([np.nan, -0.0, 0.0, -1.5, 2.5, np.inf, -np.inf, 1e-45, 3.0], np.float32)
    assert np.array_equal(host(nz.relu(dev(v))), oracle.relu(v))


def test_empty_extents(nz):
    import torch
    A = torch.zeros((0, 8), device="cuda")
    B = torch.zeros((8, 4), device="cuda")
    assert nz.gemm(A, B).shape == (0, 4)
    # K == 0: empty sum, C = act(bias)
    A = torch.zeros((3, 0), device="cuda")
    B = torch.zeros((0, 4), device="cuda")
    bias = dev(np.array([-1, 2, -3, 4], np.float32))
    out = torch.full((3, 4), 7.0, device="cuda")
    nz.gemm(A, B, bias=bias, bias_strides=(0, 1), relu=True, out=out)
    assert np.array_equal(host(out), np.tile(np.array([0, 2, 0, 4], np.float32), (3, 1)))


def test_invalid_arguments_are_rejected_without_launching(nz):
    import ctypes as C
    import torch
    A = torch.zeros((4, 4), device="cuda")
    d = nz.GemmDesc()
    d.A = d.B = d.C = A.data_ptr()
    d.M = d.N = d.K = 4
    d.lda = d.ldb = d.ldc = 4
    d.batch_n = d.batch_c = 1
    lib = nz.load()
    assert lib.nzhip_gemm(C.byref(d), None) == 0
    d.lda = 2
    assert lib.nzhip_gemm(C.byref(d), None) == -1 and b"leading dimension" in lib.nzhip_last_error()
    d.lda = 4
    d.activation = 9
    assert lib.nzhip_gemm(C.byref(d), None) == -1
    d.activation = 0
    d.batch_n = 0
    assert lib.nzhip_gemm(C.byref(d), None) == -1
    d.batch_n = 1
    d.A = None
    assert lib.nzhip_gemm(C.byref(d), None) == -1 and b"null operand" in lib.nzhip_last_error()
    assert lib.nzhip_gemm(None, None) == -1
    torch.cuda.synchronize()


def test_config5_large_square_sampled_rows(nz, oracle):
    n = 8192
    A = oracle.fill((n, n), 5, "normal", 0.0, 1.0 / np.sqrt(n))
    B = oracle.fill((n, n), 1005, "normal", 0.0, 1.0 / np.sqrt(n))
    got = nz.gemm(dev(A), dev(B))
    rows = np.random.default_rng(5).choice(n, size=64, replace=False)
    rows.sort()
    got_rows = host(got[rows.tolist()])
    truth = np.empty((64, n), np.float64)
    for i, r in enumerate(rows):
        _, t = oracle.gemm_rows(A, B, int(r), 1, want32=False)
        truth[i] = t[0]
    check_tolerance(oracle, got_rows, truth, "G2 sampled rows")
    # size-independent property at full size: (A*B) e_j picks column j -- multiply by the identity
    # on the right reproduces f16(A) exactly
    I = dev(np.eye(n, dtype=np.float32))
    Ad = dev(A)
    assert np.array_equal(host(nz.gemm(Ad, I)), oracle.round_f16(A))


@pytest.mark.parametrize("M,K,N,b_trans", [(8192, 8192, 8192, False), (8192, 8192, 8192, True), (4096, 1024, 4096, True), (1000, 777, 513, False)])
def test_whole_output_at_full_size_against_torch_fp32_product(nz, M, K, N, b_trans):
    # every element of the headline product (and of the Linear and ragged configs) against an implementation that shares
    # nothing with this one: torch's fp32 matmul on the operands rounded to fp16 first. Both accumulate in fp32, in
    # different orders: 1e-5 relative in the Frobenius norm (3e-7 measured), and no element off by more than 1e-3 of the
    # largest one.
    import torch
    torch.backends.cuda.matmul.allow_tf32 = False
    g = torch.Generator(device="cuda").manual_seed(M + K + N)
    A = torch.randn(M, K, device="cuda", generator=g) / np.sqrt(K)
    B = torch.randn((N, K) if b_trans else (K, N), device="cuda", generator=g)
    got = nz.gemm(A, B, b_trans=b_trans)
    Br = B.half().float()
    want = torch.matmul(A.half().float(), Br.t() if b_trans else Br)
    diff = got - want
    assert float(diff.norm() / want.norm()) < 1e-5
    assert float(diff.abs().max()) < 1e-3 * float(want.abs().max())
    del got, want, diff, Br
    torch.cuda.empty_cache()


def test_config5_batched_1024(nz, oracle):
    # [8,16,1024,1024] x [8,16,1024,1024] over (N,C); three seeded batch members checked in full
    import torch
    shape = (8, 16, 1024, 1024)
    A = oracle.fill(shape, 6, "normal", 0.0, 1.0 / 32.0)
    B = oracle.fill(shape, 1006, "normal", 0.0, 1.0 / 32.0)
    got = nz.tensorcore_gemm(dev(A), dev(B))
    for (i, j) in [(0, 0), (3, 7), (7, 15)]:
        check_tolerance(oracle, host(got[i, j]), oracle.gemm_f64(A[i, j], B[i, j]), f"GB[{i},{j}]")
    del got
    torch.cuda.empty_cache()
