// Entry points of the GEMM path and the unfused lowering kernels (im2col, col2im, broadcast
// add, ReLU). The unfused kernels exist so that a graph built node by node
// (Img2Col -> MatMul -> Add -> Col2Img -> ReLU, src/Model.cu:244-263 of the reference) keeps
// working; the fused route is nzhip_conv2d_forward / nzhip_gemm with bias and activation.
#include <hip/hip_runtime.h>

#include <cstdlib>

#include "nzhip_internal.h"

namespace nzhip {

typedef float floatx4 __attribute__((ext_vector_type(4)));

static inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }
static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

static int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? NZHIP_OK : set_hip_error(e, what);
}

// ---- im2col (img2colKernel, src/OperationKernels.cu:1308-1328) -----------------------------
// One thread per output element, column index fastest so the writes of a wave are
// contiguous; 32-bit index math per image, 64-bit only for the image base.
__global__ __launch_bounds__(256) void im2col_kernel(float* __restrict__ out, const float* __restrict__ in,
                                                     int H_out, int W_out, int C, int K_h, int K_w, int stride,
                                                     int pad, int H_in, int W_in) {
    const int CKK = C * K_h * K_w;
    const long per = (long)H_out * W_out * CKK;
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= per) return;
    const int b = blockIdx.y;
    const int pix = (int)(idx / CKK), q = (int)(idx % CKK);
    const int c = q / (K_h * K_w), rs = q % (K_h * K_w);
    const int h = (pix / W_out) * stride - pad + rs / K_w;
    const int w = (pix % W_out) * stride - pad + rs % K_w;
    float v = 0.f;
    if (h >= 0 && h < H_in && w >= 0 && w < W_in) v = in[((long)b * C + c) * H_in * W_in + (long)h * W_in + w];
    out[(long)b * per + idx] = v;
}

// ---- col2im (col2imgKernel, :1364-1376): per-image transpose [HW, O] -> [O, HW] through LDS --
__global__ __launch_bounds__(256) void col2im_kernel(float* __restrict__ out, const float* __restrict__ in, int HW,
                                                     int O) {
    __shared__ float tile[32][33];
    const int b = blockIdx.z;
    const float* src = in + (long)b * HW * O;
    float* dst = out + (long)b * HW * O;
    const int p0 = blockIdx.x * 32, o0 = blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;   // 32 x 8
#pragma unroll
    for (int r = 0; r < 32; r += 8) {
        const int p = p0 + ty + r, o = o0 + tx;
        tile[ty + r][tx] = (p < HW && o < O) ? src[(long)p * O + o] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 32; r += 8) {
        const int o = o0 + ty + r, p = p0 + tx;
        if (o < O && p < HW) dst[(long)o * HW + p] = tile[tx][ty + r];
    }
}

// ---- broadcast add (MatrixAddKernel, :12-24, offsets of TensorOperations.cuh:793-807) -------
__global__ __launch_bounds__(256) void add_bcast_kernel(float* __restrict__ out, const float* __restrict__ a,
                                                        const float* __restrict__ b, long hw, int Cc, long o_sn,
                                                        long o_sc, long a_sn, long a_sc, long b_sn, long b_sc,
                                                        int vec) {
    const int i = blockIdx.y / Cc, j = blockIdx.y % Cc;
    float* o_m = out + i * o_sn + j * o_sc;
    const float* a_m = a + i * a_sn + j * a_sc;
    const float* b_m = b + i * b_sn + j * b_sc;
    const long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (vec) {
        if (t * 4 < hw) {
            const floatx4 x = reinterpret_cast<const floatx4*>(a_m)[t], y = reinterpret_cast<const floatx4*>(b_m)[t];
            reinterpret_cast<floatx4*>(o_m)[t] = x + y;
        }
    } else if (t < hw) {
        o_m[t] = a_m[t] + b_m[t];
    }
}

// ---- ReLU (RectifiedLinearUnitKernel, :230-235) ---------------------------------------------
__global__ __launch_bounds__(256) void relu_kernel(float* __restrict__ out, const float* __restrict__ in, long n,
                                                   int vec) {
    const long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (vec) {
        if (t * 4 + 3 < n) {
            floatx4 x = reinterpret_cast<const floatx4*>(in)[t];
#pragma unroll
            for (int e = 0; e < 4; e++) x[e] = x[e] > 0.f ? x[e] : 0.f;
            reinterpret_cast<floatx4*>(out)[t] = x;
        } else {
            for (long k = t * 4; k < n; k++) out[k] = in[k] > 0.f ? in[k] : 0.f;
        }
    } else if (t < n) {
        out[t] = in[t] > 0.f ? in[t] : 0.f;
    }
}

static int validate_gemm(const nzhip_gemm_desc& d) {
    if (d.M < 0 || d.N < 0 || d.K < 0) return set_error(NZHIP_E_INVALID, "nzhip_gemm: negative extent");
    // an operand with no elements may be null
    if ((!d.A && d.M * d.K > 0) || (!d.B && d.K * d.N > 0) || (!d.C && d.M * d.N > 0))
        return set_error(NZHIP_E_INVALID, "nzhip_gemm: null operand pointer");
    if (d.batch_n < 1 || d.batch_c < 1) return set_error(NZHIP_E_INVALID, "nzhip_gemm: batch extents must be >= 1");
    if (d.a_layout != NZHIP_LAYOUT_ROW && d.a_layout != NZHIP_LAYOUT_TRANS)
        return set_error(NZHIP_E_INVALID, "nzhip_gemm: bad a_layout %d", d.a_layout);
    if (d.b_layout != NZHIP_LAYOUT_ROW && d.b_layout != NZHIP_LAYOUT_TRANS)
        return set_error(NZHIP_E_INVALID, "nzhip_gemm: bad b_layout %d", d.b_layout);
    if (d.activation != NZHIP_ACT_NONE && d.activation != NZHIP_ACT_RELU)
        return set_error(NZHIP_E_INVALID, "nzhip_gemm: bad activation %d", d.activation);
    if (d.reserved != 0) return set_error(NZHIP_E_INVALID, "nzhip_gemm: reserved field must be 0");
    const int64_t a_min = d.a_layout == NZHIP_LAYOUT_ROW ? d.K : d.M;
    const int64_t b_min = d.b_layout == NZHIP_LAYOUT_ROW ? d.N : d.K;
    if (d.lda < a_min || d.ldb < b_min || d.ldc < d.N)
        return set_error(NZHIP_E_INVALID, "nzhip_gemm: leading dimension smaller than the row it strides (lda %lld ldb %lld ldc %lld)",
                         (long long)d.lda, (long long)d.ldb, (long long)d.ldc);
    if (d.a_stride_n < 0 || d.a_stride_c < 0 || d.b_stride_n < 0 || d.b_stride_c < 0 || d.c_stride_n < 0 ||
        d.c_stride_c < 0)
        return set_error(NZHIP_E_INVALID, "nzhip_gemm: negative batch stride");
    if (d.M > 0x3fffffff || d.N > 0x3fffffff || d.K > 0x3fffffff)
        return set_error(NZHIP_E_UNSUPPORTED, "nzhip_gemm: extent above 2^30");
    if (d.batch_n * d.batch_c > 65535)
        return set_error(NZHIP_E_UNSUPPORTED, "nzhip_gemm: more than 65535 batch members in one call");
    return NZHIP_OK;
}

__global__ __launch_bounds__(256) void fill_bias_act_kernel(nzhip_gemm_desc d) {
    // K == 0: the product is an empty sum, C = act(bias) (or act(0)).
    const long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= d.M * d.N) return;
    const int i = blockIdx.y / (int)d.batch_c, j = blockIdx.y % (int)d.batch_c;
    const long m = t / d.N, n = t % d.N;
    float x = 0.f;
    if (d.bias) x += d.bias[i * d.bias_stride_n + j * d.bias_stride_c + m * d.bias_stride_row + n * d.bias_stride_col];
    if (d.activation == NZHIP_ACT_RELU) x = x > 0.f ? x : 0.f;
    d.C[i * d.c_stride_n + j * d.c_stride_c + m * d.ldc + n] = x;
}

}  // namespace nzhip

using namespace nzhip;

extern "C" {

int nzhip_gemm(const nzhip_gemm_desc* desc, void* stream) {
    if (!desc) return set_error(NZHIP_E_INVALID, "nzhip_gemm: null descriptor");
    const nzhip_gemm_desc& d = *desc;
    if (int rc = validate_gemm(d)) return rc;
    if (d.M == 0 || d.N == 0) return NZHIP_OK;
    hipStream_t s = as_stream(stream);
    if (d.K == 0) {
        dim3 grid((unsigned)((d.M * d.N + 255) / 256), (unsigned)(d.batch_n * d.batch_c));
        hipLaunchKernelGGL(fill_bias_act_kernel, grid, dim3(256), 0, s, d);
        return check_launch("fill_bias_act_kernel");
    }
    if (gemm_skinny_applicable(d)) return gemm_skinny_dispatch(d, s);
    // NZHIP_GEMM_ROUTE=fused|h16 overrides the route choice (benchmarking only).
    static const char* route = getenv("NZHIP_GEMM_ROUTE");
    const bool force_fused = route && route[0] == 'f', force_h16 = route && route[0] == 'h';
    if (!force_fused && (force_h16 || gemm_h16_applicable(d))) return gemm_h16_dispatch(d, s);
    return gemm_mfma_dispatch(d, s, 0);
}

/* Test hook: pick the kernel instead of letting the shape decide. tile 128 / 256: the fused
 * convert-on-load kernel with that square tile; tile 16: the two-pass fp16 route. */
int nzhip_gemm_force_tile(const nzhip_gemm_desc* desc, int tile, void* stream) {
    if (!desc) return set_error(NZHIP_E_INVALID, "nzhip_gemm: null descriptor");
    if (tile != 128 && tile != 256 && tile != 16)
        return set_error(NZHIP_E_INVALID, "nzhip_gemm_force_tile: tile must be 128, 256 or 16");
    if (int rc = validate_gemm(*desc)) return rc;
    if (desc->M == 0 || desc->N == 0 || desc->K == 0) return nzhip_gemm(desc, stream);
    if (tile == 16) return gemm_h16_dispatch(*desc, as_stream(stream));
    return gemm_mfma_dispatch(*desc, as_stream(stream), tile);
}

int nzhip_tensorcore_gemm(const float* A, const float* B, float* C, const size_t sA[4], const size_t sB[4],
                          const size_t sC[4], void* stream) {
    if (!A || !B || !C || !sA || !sB || !sC) return set_error(NZHIP_E_INVALID, "nzhip_tensorcore_gemm: null argument");
    nzhip_gemm_desc d = {};
    d.A = A;
    d.B = B;
    d.C = C;
    d.M = (int64_t)sA[2];                              // src/OperationKernels.cu:918-920
    d.N = (int64_t)sB[3];
    d.K = (int64_t)sA[3];
    d.lda = d.K;
    d.ldb = d.N;
    d.ldc = d.N;
    d.batch_n = (int64_t)sC[0];                        // :978-979
    d.batch_c = (int64_t)sC[1];
    d.a_stride_n = sA[0] > 1 ? (int64_t)(sA[1] * sA[2] * sA[3]) : 0;   // :981-984
    d.a_stride_c = sA[1] > 1 ? (int64_t)(sA[2] * sA[3]) : 0;
    d.b_stride_n = sB[0] > 1 ? (int64_t)(sB[1] * sB[2] * sB[3]) : 0;
    d.b_stride_c = sB[1] > 1 ? (int64_t)(sB[2] * sB[3]) : 0;
    d.c_stride_n = (int64_t)(sC[1] * sC[2] * sC[3]);
    d.c_stride_c = (int64_t)(sC[2] * sC[3]);
    if (d.batch_n == 0 || d.batch_c == 0) return NZHIP_OK;

    // Collapse "one shared matrix times a batch of vectors" into a single GEMM.
    // (a) N == 1, A shared, B a dense batch of K-vectors (Model::Linear: W[1,1,OUT,IN] x[N,1,IN,1]):
    //     C^T[batch, M] = X[batch, K] * A^T, i.e. rows = batch members, B operand = A given as NxK.
    const bool a_shared = sA[0] == 1 && sA[1] == 1, b_shared = sB[0] == 1 && sB[1] == 1;
    const bool b_dense = sB[0] == sC[0] && sB[1] == sC[1], a_dense = sA[0] == sC[0] && sA[1] == sC[1];
    const int64_t batch = d.batch_n * d.batch_c;
    if (batch > 1 && d.N == 1 && a_shared && b_dense) {
        nzhip_gemm_desc g = {};
        g.A = B; g.B = A; g.C = C;
        g.M = batch; g.N = d.M; g.K = d.K;
        g.lda = d.K; g.ldb = d.K; g.ldc = d.M;
        g.a_layout = NZHIP_LAYOUT_ROW; g.b_layout = NZHIP_LAYOUT_TRANS;
        g.batch_n = g.batch_c = 1;
        return nzhip_gemm(&g, stream);
    }
    // (b) M == 1, B shared, A a dense batch of row vectors: C[batch, N] = A[batch, K] * B.
    if (batch > 1 && d.M == 1 && b_shared && a_dense) {
        nzhip_gemm_desc g = {};
        g.A = A; g.B = B; g.C = C;
        g.M = batch; g.N = d.N; g.K = d.K;
        g.lda = d.K; g.ldb = d.N; g.ldc = d.N;
        g.batch_n = g.batch_c = 1;
        return nzhip_gemm(&g, stream);
    }
    if (batch > 65535) {
        // Split the outer batch axis over several launches.
        const int64_t per = 65535 / d.batch_c;
        if (per < 1) return set_error(NZHIP_E_UNSUPPORTED, "nzhip_tensorcore_gemm: c extent above 65535");
        for (int64_t i0 = 0; i0 < d.batch_n; i0 += per) {
            nzhip_gemm_desc g = d;
            g.batch_n = (d.batch_n - i0) < per ? (d.batch_n - i0) : per;
            g.A = A + i0 * d.a_stride_n;
            g.B = B + i0 * d.b_stride_n;
            g.C = C + i0 * d.c_stride_n;
            if (int rc = nzhip_gemm(&g, stream)) return rc;
        }
        return NZHIP_OK;
    }
    return nzhip_gemm(&d, stream);
}

int nzhip_im2col(float* out, const float* in, size_t H_out, size_t W_out, size_t C, size_t K_h, size_t K_w,
                 size_t stride, size_t pad, size_t H_in, size_t W_in, size_t batch, void* stream) {
    if (!out || !in) return set_error(NZHIP_E_INVALID, "nzhip_im2col: null pointer");
    if (stride == 0 || K_h == 0 || K_w == 0) return set_error(NZHIP_E_INVALID, "nzhip_im2col: zero stride or kernel extent");
    const size_t per = H_out * W_out * C * K_h * K_w;
    if (per == 0 || batch == 0) return NZHIP_OK;
    if (per > 0x7fffffffull * 256 || batch > 65535 || H_in > 0x3fffffff || W_in > 0x3fffffff)
        return set_error(NZHIP_E_UNSUPPORTED, "nzhip_im2col: extent too large");
    dim3 grid((unsigned)((per + 255) / 256), (unsigned)batch);
    hipLaunchKernelGGL(im2col_kernel, grid, dim3(256), 0, as_stream(stream), out, in, (int)H_out, (int)W_out, (int)C,
                       (int)K_h, (int)K_w, (int)stride, (int)pad, (int)H_in, (int)W_in);
    return check_launch("im2col_kernel");
}

int nzhip_col2im(float* out, const float* in, size_t H_out, size_t W_out, size_t C_out, size_t batches,
                 void* stream) {
    if (!out || !in) return set_error(NZHIP_E_INVALID, "nzhip_col2im: null pointer");
    const size_t HW = H_out * W_out;
    if (HW == 0 || C_out == 0 || batches == 0) return NZHIP_OK;
    if (HW > 0x7fffffff || (C_out + 31) / 32 > 65535 || batches > 65535)
        return set_error(NZHIP_E_UNSUPPORTED, "nzhip_col2im: extent too large");
    dim3 grid((unsigned)((HW + 31) / 32), (unsigned)((C_out + 31) / 32), (unsigned)batches);
    hipLaunchKernelGGL(col2im_kernel, grid, dim3(256), 0, as_stream(stream), out, in, (int)HW, (int)C_out);
    return check_launch("col2im_kernel");
}

int nzhip_add_broadcast(float* out, const float* a, const float* b, const size_t sO[4], const size_t sA[4],
                        const size_t sB[4], void* stream) {
    if (!out || !a || !b || !sO || !sA || !sB) return set_error(NZHIP_E_INVALID, "nzhip_add_broadcast: null argument");
    // TensorOperations.cuh:787-791: n and c broadcast, h and w must agree
    for (int i = 0; i < 2; i++)
        if (sA[i] != sB[i] && sA[i] != 1 && sB[i] != 1)
            return set_error(NZHIP_E_SHAPE, "Shapes are not broadcast compatible.");
    if (sA[2] != sB[2] || sA[3] != sB[3]) return set_error(NZHIP_E_SHAPE, "Shapes are not broadcast compatible.");
    const size_t hw = sA[2] * sA[3];
    const size_t nb = sO[0] * sO[1];
    if (hw == 0 || nb == 0) return NZHIP_OK;
    if (nb > 65535) return set_error(NZHIP_E_UNSUPPORTED, "nzhip_add_broadcast: more than 65535 (n,c) planes");
    const long o_sn = (long)(sO[1] * sO[2] * sO[3]), o_sc = (long)(sO[2] * sO[3]);
    const long a_sn = sA[0] > 1 ? (long)(sA[1] * hw) : 0, a_sc = sA[1] > 1 ? (long)hw : 0;
    const long b_sn = sB[0] > 1 ? (long)(sB[1] * hw) : 0, b_sc = sB[1] > 1 ? (long)hw : 0;
    const int vec = (hw % 4 == 0) && aligned16(out) && aligned16(a) && aligned16(b);
    const size_t threads = vec ? hw / 4 : hw;
    dim3 grid((unsigned)((threads + 255) / 256), (unsigned)nb);
    hipLaunchKernelGGL(add_bcast_kernel, grid, dim3(256), 0, as_stream(stream), out, a, b, (long)hw, (int)sO[1], o_sn,
                       o_sc, a_sn, a_sc, b_sn, b_sc, vec);
    return check_launch("add_bcast_kernel");
}

int nzhip_relu(float* out, const float* in, size_t n, void* stream) {
    if ((!out || !in) && n) return set_error(NZHIP_E_INVALID, "nzhip_relu: null pointer");
    if (n == 0) return NZHIP_OK;
    const int vec = aligned16(out) && aligned16(in);
    const size_t threads = vec ? (n + 3) / 4 : n;
    hipLaunchKernelGGL(relu_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, as_stream(stream), out, in,
                       (long)n, vec);
    return check_launch("relu_kernel");
}

}  // extern "C"
