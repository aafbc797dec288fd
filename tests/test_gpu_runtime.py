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


def test_memset_writes_the_byte_value_for_word_and_odd_sizes(nz):
    # whole fp32 words go through the library's fill kernel (the byte repeated four times as one bit pattern, NaN patterns
    # included), anything else through the runtime's memset; either way every byte of the range, and none beyond it
    import ctypes as C
    lib = nz.load()
    for value, nbytes, offset in ((0x00, 4096, 0), (0xFF, 4096, 0), (0xAB, 4 * 1031, 0), (0x7F, 1001, 0), (0x3C, 64, 2)):
        p = C.c_void_p()
        nz.check(lib.nzhip_malloc(C.byref(p), nbytes + 64))
        guard = np.full(nbytes + 64, 0x55, np.uint8)
        nz.check(lib.nzhip_memcpy_h2d(p, guard.ctypes.data_as(C.c_void_p), guard.nbytes))
        nz.check(lib.nzhip_memset(C.c_void_p(p.value + 16 + offset), value, nbytes))
        got = np.empty_like(guard)
        nz.check(lib.nzhip_memcpy_d2h(got.ctypes.data_as(C.c_void_p), p, got.nbytes))
        want = guard.copy()
        want[16 + offset:16 + offset + nbytes] = value
        assert np.array_equal(got, want), (value, nbytes, offset)
        nz.check(lib.nzhip_free_async(p))


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


def test_entry_points_from_four_host_threads_at_once(nz):
    """Thread-safe entry points (the reference's singleton manager is mutex-protected, StreamManager.cuh:799-805): four
    host threads, each on its own stream, call products of every route family, a convolution through its own prepared
    handle and a chunked broadcast gradient at the same time; every result must be the single-threaded one. What is
    shared between them: the workspace pool, the per-kernel LDS limits, the error string (thread-local), the prepared
    scope (thread-local). The single-kernel route for very large products needs the GPU to itself and is not part of
    this."""
    import threading
    import torch
    rng = np.random.default_rng(101)

    def ints(shape, lo=-4, hi=5):
        return torch.from_numpy(rng.integers(lo, hi, size=shape).astype(np.float32)).cuda()

    gemms = [(300, 200, 100), (1024, 1024, 1024), (1, 4096, 4096), (2048, 1024, 2048), (64, 8192, 64), (1000, 777, 513)]
    work = []
    for M, K, N in gemms:
        A, B = ints((M, K)), ints((K, N))
        work.append(("gemm", (A, B), (A.double() @ B.double()).float()))
    x, w = ints((4, 32, 64, 64)), ints((1, 1, 32 * 9, 64), -2, 3)
    want_conv = nz.conv2d_forward(x, w, None, 3, 3, 1, 1)
    dout = ints((600, 1, 256, 1))
    want_bias = dout.sum(dim=0, keepdim=True)
    torch.cuda.synchronize()
    errors = []

    def worker(tid):
        try:
            stream = torch.cuda.Stream()
            handle = nz.Prepared()
            with torch.cuda.stream(stream):
                for rep in range(4):
                    for i in range(len(work)):
                        kind, (A, B), want = work[(i + tid) % len(work)]
                        got = nz.gemm(A, B, stream=stream)
                        stream.synchronize()
                        if not torch.equal(got, want):
                            errors.append((tid, rep, "gemm", tuple(A.shape), tuple(B.shape)))
                    y = nz.conv2d_forward(x, w, None, 3, 3, 1, 1, stream=stream, prepared_w=handle)
                    din = torch.zeros((1, 1, 256, 1), device="cuda")
                    nz.add_backward(din, dout, stream=stream)
                    stream.synchronize()
                    if not torch.equal(y, want_conv):
                        errors.append((tid, rep, "conv"))
                    if not torch.equal(din, want_bias):
                        errors.append((tid, rep, "add_backward"))
            if handle.fills() != 1:
                errors.append((tid, "fills", handle.fills()))
            handle.close()
        except Exception as e:                                        # noqa: BLE001 - reported below
            errors.append((tid, repr(e)))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors[:5]
