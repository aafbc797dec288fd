"""Conv2d layers at their real sizes (shapes of ResNet-50 and VGG-16 at batch 16, and two with rows that are not whole
16-byte pieces), forward and both gradients through the C-ABI, against an independent implementation: torch's own fp32
convolution and its autograd on the same operands rounded to fp16 first (what the kernels multiply). The oracle checks the
same entry points bit for bit on sizes it finishes in seconds; this checks the sizes the routes were tuned on — every route
choice that depends on the extents (resident weights, two chunks per step, widened rows, column-gradient chains, the folded
weight gradient, per-sample epilogues) is taken here the way a network would take it. Both parameter forms: shared weights
with a per-channel bias, and the reference's own (one weight copy per image, a bias per pixel and channel,
src/Model.cu:244-256). Tolerance: 1e-4 relative in the Frobenius norm (fp32 accumulation in another order; measured
2e-6 at worst)."""
import pytest

pytestmark = pytest.mark.gpu

N = 16
LAYERS = [  # C, H, W, O, K, stride, pad
    (3, 224, 224, 64, 7, 2, 3), (64, 56, 56, 64, 1, 1, 0), (256, 56, 56, 128, 1, 1, 0), (128, 56, 56, 128, 3, 2, 1),
    (256, 56, 56, 512, 1, 2, 0), (256, 14, 14, 256, 3, 1, 1), (512, 14, 14, 512, 3, 2, 1), (512, 7, 7, 2048, 1, 1, 0),
    (512, 7, 7, 512, 3, 1, 1), (3, 224, 224, 64, 3, 1, 1), (64, 112, 112, 128, 3, 1, 1), (256, 56, 56, 256, 3, 1, 1),
    (512, 28, 28, 512, 3, 1, 1), (512, 14, 14, 512, 3, 1, 1), (192, 35, 35, 192, 3, 1, 1), (128, 30, 30, 128, 5, 1, 2),
    (768, 17, 17, 192, 1, 1, 0)]


@pytest.fixture(scope="module")
def nz():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from neuzephyr_amd import capi
    capi.load()
    return capi


@pytest.mark.parametrize("form", ["shared", "reference"])
@pytest.mark.parametrize("C,H,W,O,K,stride,pad", LAYERS)
def test_layer_at_full_size_against_torch_convolution(nz, C, H, W, O, K, stride, pad, form):
    import torch
    import torch.nn.functional as F
    Ho, Wo = (H + 2 * pad - K) // stride + 1, (W + 2 * pad - K) // stride + 1
    reference_form = form == "reference"
    wb = N if reference_form else 1
    g = torch.Generator(device="cuda").manual_seed(C + H + O + K + stride)
    x = torch.randn(N, C, H, W, device="cuda", generator=g)
    dy = torch.randn(N, O, Ho, Wo, device="cuda", generator=g)
    w = torch.randn(wb, 1, C * K * K, O, device="cuda", generator=g) * 0.05
    bias = torch.randn((1, 1, Ho * Wo, O) if reference_form else (O,), device="cuda", generator=g)
    y = nz.conv2d_forward(x, w, bias, K, K, stride, pad, bias_strides=(O, 1) if reference_form else (0, 1), relu=False)
    dx = nz.conv2d_backward_data(torch.zeros_like(x), dy, w, K, K, stride, pad, accumulate=False)
    dw = nz.conv2d_backward_weights(torch.zeros_like(w), x, dy, K, K, stride, pad)
    torch.cuda.synchronize()

    def rounded(t):
        return t.half().float()

    def rel(a, b):
        return float((a - b).norm() / (b.norm() + 1e-30))

    badd = bias.view(Ho, Wo, O).permute(2, 0, 1)[None] if reference_form else bias.view(1, O, 1, 1)
    images = [(n, n + 1) for n in (0, N // 2, N - 1)] if wb > 1 else [(0, N)]     # per-sample weights: three of the images
    for n0, n1 in images:
        wt = rounded(w[n0 if wb > 1 else 0, 0]).view(C, K, K, O).permute(3, 0, 1, 2).contiguous().requires_grad_(True)
        xt = rounded(x[n0:n1]).requires_grad_(True)
        yt = F.conv2d(xt, wt, None, stride, pad)
        gx, gw = torch.autograd.grad(yt, (xt, wt), rounded(dy[n0:n1]))
        assert rel(y[n0:n1], yt.detach() + badd) < 1e-4, ("forward", n0)
        assert rel(dx[n0:n1], gx) < 1e-4, ("data gradient", n0)
        assert rel(dw[n0 if wb > 1 else 0, 0].view(C, K, K, O).permute(3, 0, 1, 2), gw) < 1e-4, ("weight gradient", n0)
