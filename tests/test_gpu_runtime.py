"""The runtime's allocator and stream manager through the C-ABI: memory from nzhip_malloc used by a
product on ANOTHER stream, then copied out, freed and re-issued through the runtime. The runtime only
orders work on its own stream, so the caller joins the two with nzhip_stream_wait (the stated
precondition); with it the copy must see the finished product and the re-issued block must not
disturb it."""
import ctypes as C

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


def test_product_on_a_second_stream_then_free_and_reissue_through_the_runtime(nz):
    import torch
    lib = nz.load()
    M, K, N = 2048, 4096, 2048                       # long enough (tens of microseconds) to still run at the free
    rng = np.random.default_rng(7)
    A = np.rint(rng.uniform(-4, 4, (M, K))).astype(np.float32)      # small integers: the product is exact
    B = np.rint(rng.uniform(-4, 4, (K, N))).astype(np.float32)
    want = (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32)    # |sums| < 2^24: exact in any order

    def dmalloc(nbytes):
        p = C.c_void_p()
        nz.check(lib.nzhip_malloc(C.byref(p), nbytes))
        return p

    a, b, c = dmalloc(A.nbytes), dmalloc(B.nbytes), dmalloc(M * N * 4)
    nz.check(lib.nzhip_memcpy_h2d(a, A.ctypes.data_as(C.c_void_p), A.nbytes))
    nz.check(lib.nzhip_memcpy_h2d(b, B.ctypes.data_as(C.c_void_p), B.nbytes))
    nz.check(lib.nzhip_memset(c, 0xFF, M * N * 4))               # NaN pattern
    nz.check(lib.nzhip_sync_ptr(c))                                # the other direction is the caller's job

    second = torch.cuda.Stream()                                   # default priority
    d = nz.GemmDesc()
    d.A, d.B, d.C = a.value, b.value, c.value
    d.M, d.N, d.K = M, N, K
    d.lda, d.ldb, d.ldc = K, N, N
    d.batch_n = d.batch_c = 1
    for _ in range(3):                                             # a queue of work on the second stream
        nz.check(lib.nzhip_gemm(C.byref(d), C.c_void_p(second.cuda_stream)))
    nz.check(lib.nzhip_stream_wait(C.c_void_p(second.cuda_stream)))
    got = np.empty((M, N), np.float32)
    nz.check(lib.nzhip_memcpy_d2h(got.ctypes.data_as(C.c_void_p), c, got.nbytes))   # runtime stream, after the wait
    nz.check(lib.nzhip_free_async(c))
    c2 = dmalloc(M * N * 4)                                        # the cached block comes straight back
    assert c2.value == c.value
    nz.check(lib.nzhip_memset(c2, 0, M * N * 4))
    nz.check(lib.nzhip_sync_ptr(c2))
    second.synchronize()
    assert np.array_equal(got, want)
    for p in (a, b, c2):
        nz.check(lib.nzhip_free_async(p))
    # waiting for the runtime's own stream is a no-op, a null handle means HIP's null stream
    nz.check(lib.nzhip_stream_wait(lib.nzhip_default_stream()))
    nz.check(lib.nzhip_stream_wait(None))


def test_pinned_host_operands(nz):
    # page-locked host memory is mapped into the device at the same address: the kernels take it as any operand
    # (the storage of nz::data::MappedTensor); host-memory result == device-memory result, bit for bit
    import ctypes as C
    import numpy as np
    import torch
    lib = nz.load()
    rng = np.random.default_rng(5)
    for (M, K, N) in [(64, 96, 48), (1, 300, 130), (130, 70, 257)]:
        A = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32))
        B = torch.from_numpy(rng.standard_normal((K, N)).astype(np.float32))
        bias = torch.from_numpy(rng.standard_normal((N,)).astype(np.float32))
        want = nz.gemm(A.cuda(), B.cuda(), bias=bias.cuda(), bias_strides=(0, 1), relu=True)
        out = torch.empty((M, N), dtype=torch.float32).pin_memory()
        got = nz.gemm(A.pin_memory(), B.pin_memory(), bias=bias.pin_memory(), bias_strides=(0, 1), relu=True, out=out)
        torch.cuda.synchronize()
        assert torch.equal(got, want.cpu())
    # the runtime's own host allocator
    p = C.c_void_p()
    nz.check(lib.nzhip_host_malloc(C.byref(p), 4096 * 4))
    host = (C.c_float * 4096).from_address(p.value)
    for i in range(4096):
        host[i] = float(i % 17) - 8.0
    nz.check(lib.nzhip_relu(p, p, 4096, lib.nzhip_default_stream()))
    nz.check(lib.nzhip_sync_ptr(p))
    assert all(host[i] == max(float(i % 17) - 8.0, 0.0) for i in range(4096))
    nz.check(lib.nzhip_relu(p, p, 4096, lib.nzhip_default_stream()))
    nz.check(lib.nzhip_host_free(p))                            # waits for the kernel, then releases
    q = C.c_void_p(1)
    nz.check(lib.nzhip_host_malloc(C.byref(q), 0))
    assert q.value is None
    nz.check(lib.nzhip_host_free(None))
