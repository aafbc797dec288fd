// Conv2d forward: the Model::Conv2d graph of the reference (src/Model.cu:244-263:
// Img2Col -> MatMul -> Bias -> Col2Img [-> ReLU]) as one call.
#include <hip/hip_runtime.h>

#include "nzhip_internal.h"

namespace nzhip {

// General route: column matrix in a pooled workspace, then ONE batched GEMM that computes the
// transposed product  y_b[O, HW] = w_b^T[O, CKK] * col_b^T[CKK, HW]  so that bias, activation
// and the col2im transpose (src/OperationKernels.cu:1364-1376) all happen in its epilogue and
// the result is written once, in NCHW order.
static int conv2d_via_workspace(float* y, const float* x, const float* w_ref, const float* bias, size_t N, size_t C,
                                size_t H, size_t W, size_t O, size_t K_h, size_t K_w, size_t stride, size_t pad,
                                size_t w_batch, int64_t bias_sp, int64_t bias_sc, int act, size_t H_out,
                                size_t W_out, hipStream_t s) {
    const size_t HW = H_out * W_out, CKK = C * K_h * K_w;
    // Bound the workspace: process the batch in chunks of at most ~1 GiB of column matrix.
    const size_t per_image = HW * CKK * sizeof(float);
    size_t chunk = per_image ? (size_t(1) << 30) / per_image : N;
    if (chunk < 1) chunk = 1;
    if (chunk > N) chunk = N;
    float* col = nullptr;
    if (int rc = workspace_alloc(reinterpret_cast<void**>(&col), chunk * per_image, s)) return rc;
    int rc = NZHIP_OK;
    for (size_t b0 = 0; b0 < N && rc == NZHIP_OK; b0 += chunk) {
        const size_t nb = (N - b0) < chunk ? (N - b0) : chunk;
        rc = nzhip_im2col(col, x + b0 * C * H * W, H_out, W_out, C, K_h, K_w, stride, pad, H, W, nb, s);
        if (rc) break;
        nzhip_gemm_desc g = {};
        g.A = w_ref + (w_batch > 1 ? b0 * CKK * O : 0);
        g.B = col;
        g.C = y + b0 * O * HW;
        g.M = (int64_t)O;
        g.N = (int64_t)HW;
        g.K = (int64_t)CKK;
        g.a_layout = NZHIP_LAYOUT_TRANS;   // w_ref is [CKK, O]: A^T as stored
        g.lda = (int64_t)O;
        g.b_layout = NZHIP_LAYOUT_TRANS;   // col is [HW, CKK]: B^T as stored
        g.ldb = (int64_t)CKK;
        g.ldc = (int64_t)HW;
        g.batch_n = (int64_t)nb;
        g.batch_c = 1;
        g.a_stride_n = w_batch > 1 ? (int64_t)(CKK * O) : 0;
        g.b_stride_n = (int64_t)(HW * CKK);
        g.c_stride_n = (int64_t)(O * HW);
        g.bias = bias;
        g.bias_stride_row = bias_sc;       // output row = channel
        g.bias_stride_col = bias_sp;       // output column = pixel
        g.activation = act;
        rc = nzhip_gemm(&g, s);
    }
    int rc2 = workspace_free(col, s);
    return rc ? rc : rc2;
}

}  // namespace nzhip

using namespace nzhip;

extern "C" int nzhip_conv2d_forward(float* y, const float* x, const float* w_ref, const float* bias, size_t N,
                                    size_t C, size_t H, size_t W, size_t O, size_t K_h, size_t K_w, size_t stride,
                                    size_t pad, size_t w_batch, int64_t bias_stride_pixel,
                                    int64_t bias_stride_channel, int activation, void* stream) {
    if (!y || !x || !w_ref) return set_error(NZHIP_E_INVALID, "nzhip_conv2d_forward: null pointer");
    if (stride == 0 || K_h == 0 || K_w == 0) return set_error(NZHIP_E_INVALID, "nzhip_conv2d_forward: zero stride or kernel extent");
    if (w_batch != 1 && w_batch != N) return set_error(NZHIP_E_SHAPE, "Shapes are not broadcast compatible.");
    if (activation != NZHIP_ACT_NONE && activation != NZHIP_ACT_RELU)
        return set_error(NZHIP_E_INVALID, "nzhip_conv2d_forward: bad activation %d", activation);
    if (H + 2 * pad < K_h || W + 2 * pad < K_w)
        return set_error(NZHIP_E_SHAPE, "nzhip_conv2d_forward: kernel larger than the padded input");
    const size_t H_out = (H + 2 * pad - K_h) / stride + 1, W_out = (W + 2 * pad - K_w) / stride + 1;   // Nodes.cu:605-617
    if (N == 0 || O == 0 || C == 0) return NZHIP_OK;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    return conv2d_via_workspace(y, x, w_ref, bias, N, C, H, W, O, K_h, K_w, stride, pad, w_batch, bias_stride_pixel,
                                bias_stride_channel, activation, H_out, W_out, s);
}
