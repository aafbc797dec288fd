"""nzhip_gemm_static, the GEMM entry point that allocates nothing: its results must equal
nzhip_gemm's bit for bit (same kernels, workspace in the static device array instead of the pool),
on two calls in a row with the second one smaller, for every route that uses a workspace; the
caching pool must not be touched; a product whose workspace exceeds the array is rejected."""
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


def pool_stats(nz):
    a, b, c = C.c_size_t(0), C.c_size_t(0), C.c_size_t(0)
    nz.check(nz.load().nzhip_allocator_stats(C.byref(a), C.byref(b), C.byref(c)))
    return a.value, b.value, c.value


def rand(shape, seed):
    import torch
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.rand(shape, generator=g) * 2 - 1).cuda()


# (first call, second smaller call) per workspace-using route of nzhip_gemm
ROUTES = {
    "split contraction": [(256, 4096, 256), (128, 2048, 192)],
    "streamed skinny": [(1, 4096, 4096), (1, 1024, 512)],
    "two-pass fp16": [(3072, 768, 3072), (2000, 800, 2000)],
    "padded operand copies": [(1000, 777, 513), (333, 331, 335)],
    "no workspace": [(300, 100, 200), (17, 33, 15)],
}


@pytest.mark.parametrize("route", sorted(ROUTES))
def test_static_entry_matches_pooled_entry_on_two_calls_in_a_row(nz, oracle, route):
    import torch
    cases = []
    for idx, (M, K, N) in enumerate(ROUTES[route]):
        A, B = rand((M, K), 10 + idx), rand((K, N), 20 + idx)
        bias = rand((N,), 30 + idx)
        want = nz.gemm(A, B, bias=bias, bias_strides=(0, 1), relu=(idx == 1))
        cases.append((A, B, bias, want, idx == 1))
    torch.cuda.synchronize()
    before = pool_stats(nz)
    outs = []
    for A, B, bias, want, relu in cases:            # back to back on one stream, nothing in between
        out = torch.full_like(want, float("nan"))
        nz.gemm(A, B, bias=bias, bias_strides=(0, 1), relu=relu, out=out, static=True)
        outs.append(out)
    torch.cuda.synchronize()
    assert pool_stats(nz) == before, "the static entry point went to the caching pool"
    for (A, B, bias, want, relu), out in zip(cases, outs):
        assert torch.equal(out, want), f"{route} {tuple(A.shape)} x {tuple(B.shape)}"
    # and the result itself against the oracle (fp64 accumulation of the fp16-rounded operands)
    A, B, bias, want, relu = cases[1]
    if A.shape[0] * B.shape[1] * A.shape[1] <= 2 ** 28:
        truth = oracle.gemm_f64(A.cpu().numpy(), B.cpu().numpy()) + bias.cpu().numpy()[None, :].astype(np.float64)
        truth = np.maximum(truth, 0) if relu else truth
        rms = float(np.sqrt(np.mean(truth ** 2))) or 1.0
        mr, fr = oracle.errors(outs[1].cpu().numpy(), truth, rms)
        assert mr <= 1e-3 and fr <= 1e-4, (mr, fr)


def test_static_entry_rejects_a_workspace_beyond_its_array(nz):
    import torch
    n = 4096                                           # two-pass route: 2 * 4096 * 4096 fp16 = 64 MiB
    assert nz.load().nzhip_static_scratch_bytes() == 32 << 20
    A, B = rand((n, n), 1), rand((n, n), 2)
    out = torch.zeros((n, n), device="cuda")
    with pytest.raises(nz.NzHipError) as e:
        nz.gemm(A, B, out=out, static=True)
    assert e.value.status == -3 and "static scratch" in e.value.message
    torch.cuda.synchronize()
    assert not out.any(), "nothing may be enqueued for a rejected call"
    # the next call is unaffected
    a, b = rand((256, 4096), 3), rand((4096, 256), 4)
    got = torch.empty((256, 256), device="cuda")
    nz.gemm(a, b, out=got, static=True)
    assert torch.equal(got, nz.gemm(a, b))
