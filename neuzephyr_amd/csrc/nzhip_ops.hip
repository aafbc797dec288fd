// Entry points of the GEMM path and the unfused lowering kernels (im2col, col2im, broadcast
// add, ReLU). The unfused kernels exist so that a graph built node by node
// (Img2Col -> MatMul -> Add -> Col2Img -> ReLU, src/Model.cu:244-263 of the reference) keeps
// working; the fused route is nzhip_conv2d_forward / nzhip_gemm with bias and activation.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
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

// The same with four consecutive column indices per thread and one 16-byte store (C*K_h*K_w a
// multiple of 4, 16-byte aligned output): a quarter of the store instructions and index divisions.
__global__ __launch_bounds__(256) void im2col_vec4_kernel(float* __restrict__ out, const float* __restrict__ in,
                                                          int H_out, int W_out, int C, int K_h, int K_w, int stride,
                                                          int pad, int H_in, int W_in) {
    const int CKK = C * K_h * K_w, KK = K_h * K_w;
    const long per = (long)H_out * W_out * CKK;
    const long idx = ((long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (idx >= per) return;
    const int b = blockIdx.y;
    const int pix = (int)(idx / CKK), q = (int)(idx % CKK);    // q % 4 == 0 and CKK % 4 == 0: all four in this row
    int c = q / KK, rs = q % KK;
    const int h0 = (pix / W_out) * stride - pad, w0 = (pix % W_out) * stride - pad;
    const float* img = in + (long)b * C * H_in * W_in;
    floatx4 v;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const int h = h0 + rs / K_w, w = w0 + rs % K_w;
        v[e] = (h >= 0 && h < H_in && w >= 0 && w < W_in) ? img[((long)c * H_in + h) * W_in + w] : 0.f;
        if (++rs == KK) {
            rs = 0;
            c++;
        }
    }
    *reinterpret_cast<floatx4*>(out + (long)b * per + idx) = v;
}

// Stride 1: a workgroup takes 64 adjacent output pixels of one row (or, for images narrower than 64
// pixels, the whole rows that make up at most 64 pixels) and 32 channels, reads the input rows they
// touch once (coalesced along w) into LDS and writes, per pixel, its contiguous run of 32*K_h*K_w column
// entries with 16-byte stores (for 3x3 that is 1152 bytes: whole 128-byte lines). The scattered 4-byte
// global reads of the kernels above (a wave touches 64 channel planes per instruction) are what bounds
// them.
constexpr int I2C_PX = 64, I2C_CH = 32, I2C_MAXK = 5, I2C_ROW = I2C_PX + I2C_MAXK;   // floats per staged row
constexpr int I2C_LDS = I2C_CH * I2C_MAXK * I2C_ROW;                                  // floats of staging space
// KH, KW > 0: kernel extents known at compile time (the index divisions become multiplications).
// rpw: output rows per workgroup (1 when a row has several 64-pixel segments).
template <int KH, int KW>
__global__ __launch_bounds__(256) void im2col_rows_kernel(float* __restrict__ out, const float* __restrict__ in,
                                                          int H_out, int W_out, int C, int K_h_rt, int K_w_rt, int pad,
                                                          int H_in, int W_in, int segs, int rpw) {
    __shared__ float rows[I2C_LDS];
    const int K_h = KH > 0 ? KH : K_h_rt, K_w = KW > 0 ? KW : K_w_rt;
    const int KK = K_h * K_w, CKK = C * KK;
    const int seg = blockIdx.x % segs, ho0 = (blockIdx.x / segs) * rpw;
    const int c0 = blockIdx.y * I2C_CH, b = blockIdx.z;
    const int nch = (C - c0) < I2C_CH ? (C - c0) : I2C_CH;
    const int wo0 = seg * I2C_PX;
    const int wpx = (W_out - wo0) < I2C_PX ? (W_out - wo0) : I2C_PX;      // output pixels per row of this workgroup
    const int nrow = (H_out - ho0) < rpw ? (H_out - ho0) : rpw;           // output rows of this workgroup
    const int span = wpx + K_w - 1;                              // input columns wo0 - pad .. wo0 - pad + span - 1
    const int rt = nrow + K_h - 1;                               // input rows ho0 - pad .. ho0 - pad + rt - 1
    const float* img = in + ((long)b * C + c0) * H_in * W_in;
    for (int e = threadIdx.x; e < nch * rt * span; e += 256) {
        const int col = e % span, r = (e / span) % rt, c = e / (span * rt);
        const int h = ho0 - pad + r, w = wo0 - pad + col;
        rows[(c * rt + r) * span + col] = (h >= 0 && h < H_in && w >= 0 && w < W_in) ? img[((long)c * H_in + h) * W_in + w] : 0.f;
    }
    __syncthreads();
    const int run4 = nch * KK / 4;                               // 16-byte pieces per pixel (nch*KK is a multiple of 4)
    const int npx = nrow * wpx;                                  // rpw > 1 only with whole rows: pixels stay contiguous
    float* dst = out + ((long)b * H_out * W_out + (long)ho0 * W_out + wo0) * CKK + (long)c0 * KK;
    for (int e = threadIdx.x; e < npx * run4; e += 256) {
        const int px = e / run4, q4 = e % run4;
        const int pr = px / wpx, pw = px % wpx;
        int c = (q4 * 4) / KK, rs = (q4 * 4) % KK;
        floatx4 v;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            v[j] = rows[(c * rt + pr + rs / K_w) * span + pw + rs % K_w];
            if (++rs == KK) {
                rs = 0;
                c++;
            }
        }
        *reinterpret_cast<floatx4*>(dst + (long)px * CKK + q4 * 4) = v;
    }
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

// ---- backward element-wise kernels -----------------------------------------------------------
// ReLUBackwardKernel (src/OperationKernels.cu:242-248): dx = x > 0 ? dy : 0 (overwrites dx).
__global__ __launch_bounds__(256) void relu_backward_kernel(float* __restrict__ dx, const float* __restrict__ x,
                                                            const float* __restrict__ dy, long n, int vec) {
    const long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (vec) {
        if (t * 4 + 3 < n) {
            const floatx4 a = reinterpret_cast<const floatx4*>(x)[t], g = reinterpret_cast<const floatx4*>(dy)[t];
            floatx4 o;
#pragma unroll
            for (int e = 0; e < 4; e++) o[e] = a[e] > 0.f ? g[e] : 0.f;
            reinterpret_cast<floatx4*>(dx)[t] = o;
        } else {
            for (long k = t * 4; k < n; k++) dx[k] = x[k] > 0.f ? dy[k] : 0.f;
        }
    } else if (t < n) {
        dx[t] = x[t] > 0.f ? dy[t] : 0.f;
    }
}

// gradCopyKernel over every (n,c) of the output (src/Nodes.cu:107-121, OperationKernels.cu:1230-1236):
// din[n or 0][c or 0][:] += dout[n][c][:]. One thread owns one element of din and adds the members
// that map onto it in ascending (n,c) order, so the sum does not depend on scheduling.
__global__ __launch_bounds__(256) void grad_reduce_kernel(float* __restrict__ din, const float* __restrict__ dout,
                                                          long hw, int in_n, int in_c, int out_n, int out_c) {
    const long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= hw) return;
    const int i0 = blockIdx.y / in_c, j0 = blockIdx.y % in_c;
    float* dst = din + ((long)i0 * in_c + j0) * hw + t;
    float acc = *dst;
    const int i_lo = in_n > 1 ? i0 : 0, i_hi = in_n > 1 ? i0 + 1 : out_n;
    const int j_lo = in_c > 1 ? j0 : 0, j_hi = in_c > 1 ? j0 + 1 : out_c;
    for (int i = i_lo; i < i_hi; i++)
        for (int j = j_lo; j < j_hi; j++) acc += dout[((long)i * out_c + j) * hw + t];
    *dst = acc;
}

// The same sum when hundreds of members map onto one element (the bias of a Linear layer: one vector against a batch
// of thousands): a chain of that length in one thread is a millisecond of load latency. The members are cut into chunks;
// a thread adds one chunk in ascending order, eight loads in flight, into a partial sum, and a second kernel adds the
// partial sums onto din in ascending chunk order. Fixed order, but not the single chain of the kernel above, so it is
// used only from GRAD_CHUNK_MIN members on. Members of one element are `stride` floats apart.
constexpr int GRAD_CHUNK_MIN = 128;

__global__ __launch_bounds__(256) void grad_partial_kernel(float* __restrict__ partial, const float* __restrict__ dout, long hw,
                                                           int in_n, int in_c, int out_n, int out_c, int chunk) {
    const long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= hw) return;
    const int i0 = blockIdx.y / in_c, j0 = blockIdx.y % in_c;
    // members in ascending (n, c): n and c both broadcast -> consecutive planes; only c -> the planes of image i0;
    // only n -> plane j0 of every image
    const long members = (in_n > 1 ? 1L : out_n) * (in_c > 1 ? 1L : out_c);
    const long first = ((long)(in_n > 1 ? i0 : 0) * out_c + (in_c > 1 ? j0 : 0)) * hw;
    const long stride = (in_c > 1 ? (long)out_c : 1L) * hw;
    const long m_lo = (long)blockIdx.z * chunk, m_hi = m_lo + chunk < members ? m_lo + chunk : members;
    const float* src = dout + first + m_lo * stride + t;
    float acc = 0.f;
    long m = m_lo;
    for (; m + 8 <= m_hi; m += 8, src += 8 * stride) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = src[u * stride];
#pragma unroll
        for (int u = 0; u < 8; u++) acc += v[u];
    }
    for (; m < m_hi; m++, src += stride) acc += *src;
    partial[((long)blockIdx.y * gridDim.z + blockIdx.z) * hw + t] = acc;
}

__global__ __launch_bounds__(256) void grad_partial_sum_kernel(float* __restrict__ din, const float* __restrict__ partial, long hw,
                                                               int chunks) {
    const long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= hw) return;
    float acc = din[(long)blockIdx.y * hw + t];
    const float* src = partial + (long)blockIdx.y * chunks * hw + t;
    int p = 0;
    for (; p + 8 <= chunks; p += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = src[(long)(p + u) * hw];
#pragma unroll
        for (int u = 0; u < 8; u++) acc += v[u];
    }
    for (; p < chunks; p++) acc += src[(long)p * hw];
    din[(long)blockIdx.y * hw + t] = acc;
}

__global__ __launch_bounds__(256) void fill_kernel(float* __restrict__ data, float value, long n, int vec) {
    const long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (vec) {
        if (t * 4 + 3 < n) {
            const floatx4 v = {value, value, value, value};
            reinterpret_cast<floatx4*>(data)[t] = v;
        } else {
            for (long k = t * 4; k < n; k++) data[k] = value;
        }
    } else if (t < n) {
        data[t] = value;
    }
}

// img2colBackwardKernel (src/OperationKernels.cu:1337-1355) as a gather: one thread owns one image
// gradient element and adds the column-matrix gradient entries that were copied from it, in
// ascending pixel order (the order in which the reference's element index visits them); no atomics.
__global__ __launch_bounds__(256) void im2col_backward_kernel(float* __restrict__ dx, const float* __restrict__ dcol,
                                                              int H_out, int W_out, int C, int K_h, int K_w,
                                                              int stride, int pad, int H_in, int W_in) {
    const long per_img = (long)C * H_in * W_in;
    const long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= per_img) return;
    const int b = blockIdx.y;
    const int c = (int)(t / ((long)H_in * W_in));
    const int h = (int)((t / W_in) % H_in), w = (int)(t % W_in);
    const int CKK = C * K_h * K_w;
    const float* col = dcol + (long)b * H_out * W_out * CKK + (long)c * K_h * K_w;
    float acc = dx[(long)b * per_img + t];
    // ho*stride - pad + r == h with 0 <= r < K_h  <=>  ho in [ceil((h+pad-K_h+1)/stride), (h+pad)/stride]
    const int ho_lo = h + pad - K_h + 1 > 0 ? (h + pad - K_h + 1 + stride - 1) / stride : 0;
    const int ho_hi = (h + pad) / stride < H_out - 1 ? (h + pad) / stride : H_out - 1;
    const int wo_lo = w + pad - K_w + 1 > 0 ? (w + pad - K_w + 1 + stride - 1) / stride : 0;
    const int wo_hi = (w + pad) / stride < W_out - 1 ? (w + pad) / stride : W_out - 1;
    for (int ho = ho_lo; ho <= ho_hi; ho++) {
        const int r = h + pad - ho * stride;
        for (int wo = wo_lo; wo <= wo_hi; wo++) {
            const int sx = w + pad - wo * stride;
            acc += col[((long)ho * W_out + wo) * CKK + r * K_w + sx];
        }
    }
    dx[(long)b * per_img + t] = acc;
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

// ---- split-k for few-tile, long-contraction GEMMs ---------------------------------------------
// C = act(bias + sum over chunks s of P[s]). Eight threads share an output: thread q adds the
// chunks of its contiguous eighth in ascending order, then the eight partial sums are added in
// ascending q, so the result depends on the number of chunks only, never on scheduling.
// blockIdx.y is the batch member (n); its chunks are P[n][s][M][N].
__global__ __launch_bounds__(256) void splitk_reduce_kernel(nzhip_gemm_desc d, const float* __restrict__ P, int S) {
    __shared__ float part[8][32];
    const long mn = d.M * d.N;
    const long bn = blockIdx.y;
    P += bn * S * mn;
    const int q = threadIdx.x >> 5, tl = threadIdx.x & 31;          // a wave reads two chunk rows of 32 outputs
    const long t = (long)blockIdx.x * 32 + tl;
    const int per = (S + 7) / 8, s0 = q * per, s1 = s0 + per < S ? s0 + per : S;
    float x = 0.f;
    if (t < mn)
        for (int s = s0; s < s1; s++) x += P[(long)s * mn + t];
    part[q][tl] = x;
    __syncthreads();
    if (q != 0 || t >= mn) return;
#pragma unroll
    for (int k = 1; k < 8; k++) x += part[k][tl];
    const long m = t / d.N, n = t % d.N;
    if (d.bias) x += d.bias[bn * d.bias_stride_n + m * d.bias_stride_row + n * d.bias_stride_col];
    if (d.activation == NZHIP_ACT_RELU) x = x > 0.f ? x : 0.f;
    d.C[bn * d.c_stride_n + m * d.ldc + n] = x;
}

// Very few outputs and many chunks (a Linear layer with a huge fan-in): one wave per output. Lane l adds
// chunks l, l + 64, ... in ascending order, then the 64 sums are added in a fixed shuffle tree.
__global__ __launch_bounds__(256) void splitk_reduce_wave_kernel(nzhip_gemm_desc d, const float* __restrict__ P, int S) {
    const long mn = d.M * d.N;
    const long bn = blockIdx.y;
    P += bn * S * mn;
    const int lane = threadIdx.x & 63;
    const long t = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= mn) return;                                          // uniform over the wave
    float x = 0.f;
    for (int s = lane; s < S; s += 64) x += P[(long)s * mn + t];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) x += __shfl_down(x, off);
    if (lane != 0) return;
    const long m = t / d.N, n = t % d.N;
    if (d.bias) x += d.bias[bn * d.bias_stride_n + m * d.bias_stride_row + n * d.bias_stride_col];
    if (d.activation == NZHIP_ACT_RELU) x = x > 0.f ? x : 0.f;
    d.C[bn * d.c_stride_n + m * d.ldc + n] = x;
}

// The same sum for few chunks and many outputs: one thread per output adds its chunks in ascending
// order (coalesced along the outputs).
__global__ __launch_bounds__(256) void splitk_reduce_wide_kernel(nzhip_gemm_desc d, const float* __restrict__ P, int S) {
    const long mn = d.M * d.N;
    const long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= mn) return;
    const long bn = blockIdx.y;
    P += bn * S * mn;
    float x = 0.f;
    for (int s = 0; s < S; s++) x += P[(long)s * mn + t];
    const long m = t / d.N, n = t % d.N;
    if (d.bias) x += d.bias[bn * d.bias_stride_n + m * d.bias_stride_row + n * d.bias_stride_col];
    if (d.activation == NZHIP_ACT_RELU) x = x > 0.f ? x : 0.f;
    d.C[bn * d.c_stride_n + m * d.ldc + n] = x;
}


// ---- operands that do not allow 16-byte loads ----------------------------------------------------
// Rows that start off a 16-byte boundary or whose contiguous extent is not a multiple of 4 (1000 x 777 x 513)
// make the fused kernel load element by element, which more than halves the rate at which a CU takes
// tiles in. For a product big enough to notice, such an operand is first copied into a workspace with the
// same layout and rows padded with zeros to a multiple of 4 elements (one launch for both operands).
struct RepackOperand {
    const float* src;
    float* dst;
    long rows, cols, ld_src, ld_dst;          // rows == 0: nothing to do
};

__global__ __launch_bounds__(256) void repack_pair_kernel(const RepackOperand a, const RepackOperand b) {
    const RepackOperand& q = blockIdx.y ? b : a;
    const long per_row = q.ld_dst / 4, total = q.rows * per_row;
    for (long idx = (long)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (long)gridDim.x * 256) {
        const long r = idx / per_row, c = (idx - r * per_row) * 4;
        const float* src = q.src + r * q.ld_src + c;
        floatx4 v;
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = c + e < q.cols ? src[e] : 0.f;
        *reinterpret_cast<floatx4*>(q.dst + r * q.ld_dst + c) = v;
    }
}

}  // namespace nzhip

using namespace nzhip;

static int gemm_routed(const nzhip_gemm_desc& d, hipStream_t s, int padded = 0);

// Returns NZHIP_OK and sets *done when the product was computed from padded copies; leaves *done false when
// the copies would not pay (or the workspace is not to be had) and the caller goes on with the operands as given.
static int gemm_try_repacked(const nzhip_gemm_desc& d, hipStream_t s, bool* done) {
    *done = false;
    if (d.batch_n * d.batch_c != 1) return NZHIP_OK;
    const bool a_trans = d.a_layout == NZHIP_LAYOUT_TRANS, b_trans = d.b_layout == NZHIP_LAYOUT_TRANS;
    const int64_t a_rows = a_trans ? d.K : d.M, a_cols = a_trans ? d.M : d.K;
    const int64_t b_rows = b_trans ? d.N : d.K, b_cols = b_trans ? d.K : d.N;
    const bool a_ok = gemm_operand_vec_legal(d.A, d.lda, a_cols, 0, 0), b_ok = gemm_operand_vec_legal(d.B, d.ldb, b_cols, 0, 0);
    if (a_ok && b_ok) return NZHIP_OK;
    const int64_t a_ld = (a_cols + 3) / 4 * 4, b_ld = (b_cols + 3) / 4 * 4;
    const size_t a_bytes = a_ok ? 0 : (size_t)a_rows * a_ld * sizeof(float), b_bytes = b_ok ? 0 : (size_t)b_rows * b_ld * sizeof(float);
    nzhip_gemm_desc g = d;
    const int padded = (a_ok ? 0 : 1) | (b_ok ? 0 : 2);
    // stand-in addresses for the cost estimate: only alignment and leading dimensions matter to it
    if (!a_ok) { g.A = nullptr; g.lda = a_ld; }
    if (!b_ok) { g.B = nullptr; g.ldb = b_ld; }
    const double copy_us = 5.0 + 2.0 * (double)(a_bytes + b_bytes) / 3e6;      // launch and latency of the copy kernel, then its traffic
    if (gemm_fused_plan(g, padded).cost_us + copy_us >= 0.9 * gemm_fused_plan(d).cost_us) return NZHIP_OK;   // two plans, ~50 estimates each
    const size_t a_off = (a_bytes + 255) & ~(size_t)255;
    char* ws = nullptr;
    if (workspace_alloc(reinterpret_cast<void**>(&ws), a_off + b_bytes, s) != NZHIP_OK) return NZHIP_OK;   // no room: as given
    RepackOperand ra = {d.A, reinterpret_cast<float*>(ws), a_ok ? 0 : a_rows, a_cols, d.lda, a_ld};
    RepackOperand rb = {d.B, reinterpret_cast<float*>(ws + a_off), b_ok ? 0 : b_rows, b_cols, d.ldb, b_ld};
    if (!a_ok) g.A = ra.dst;
    if (!b_ok) g.B = rb.dst;
    const long units = std::max(ra.rows * (ra.ld_dst / 4), rb.rows * (rb.ld_dst / 4));
    const unsigned blocks = (unsigned)std::min<long>((units + 255) / 256, 4096);
    hipLaunchKernelGGL(repack_pair_kernel, dim3(blocks, 2), dim3(256), 0, s, ra, rb);
    int rc = check_launch("repack_pair_kernel");
    if (rc == NZHIP_OK) rc = gemm_routed(g, s, padded);
    const int rc2 = workspace_free(ws, s);
    *done = true;
    return rc ? rc : rc2;
}

extern "C" {

int nzhip_gemm(const nzhip_gemm_desc* desc, void* stream) {
    if (!desc) return set_error(NZHIP_E_INVALID, "nzhip_gemm: null descriptor");
    if (int rc = validate_gemm(*desc)) return rc;
    if (desc->M == 0 || desc->N == 0) return NZHIP_OK;
    return gemm_routed(*desc, as_stream(stream));
}

}  // extern "C"

namespace nzhip {
int gemm_padded_rows(const nzhip_gemm_desc& d, int padded, hipStream_t stream) {
    if (int rc = validate_gemm(d)) return rc;
    if (d.M == 0 || d.N == 0) return NZHIP_OK;
    return gemm_routed(d, stream, padded);
}
}  // namespace nzhip

// The route choice behind nzhip_gemm, for a validated descriptor with M, N > 0.
static int gemm_routed(const nzhip_gemm_desc& d, hipStream_t s, int padded) {
    if (d.K == 0) {
        dim3 grid((unsigned)((d.M * d.N + 255) / 256), (unsigned)(d.batch_n * d.batch_c));
        hipLaunchKernelGGL(fill_bias_act_kernel, grid, dim3(256), 0, s, d);
        return check_launch("fill_bias_act_kernel");
    }
    if (gemm_thin_applicable(d)) return gemm_thin_dispatch(d, s);
    if (gemm_skinny_applicable(d)) return gemm_skinny_dispatch(d, s);
    // Products that leave CUs idle with 128 x 128 tiles (weight gradients with K = batch x pixels, mid-size
    // products): smaller tiles, or the contraction cut into chunks that run as a batch into a workspace and are
    // then added in order, whichever the cost model in gemm_fused_plan prefers. A chunk keeps at least 512 of the
    // contraction when loads are vectorised and 128 otherwise. A batch over n alone (batch_c == 1: shared-weight
    // layers, the conv column-matrix route) splits the same way; its chunks take the c dimension of the launch.
    static const char* route = getenv("NZHIP_GEMM_ROUTE");         // fused | h16: overrides the route choice (benchmarking only)
    const bool force_fused = route && route[0] == 'f', force_h16 = route && route[0] == 'h';
    static const char* coop_env = getenv("NZHIP_H16_COOP");              // 0: never the single-kernel route (benchmarking only)
    const bool allow_coop = !(coop_env && atoi(coop_env) == 0);
    if (!force_fused && allow_coop && gemm_h16_coop_applicable(d)) return gemm_h16_coop_dispatch(d, s);
    if (!force_fused && (force_h16 || gemm_h16_applicable(d))) return gemm_h16_dispatch(d, s);
    {
        static const char* repack_env = getenv("NZHIP_REPACK");          // 0: never copy operands (benchmarking only)
        bool done = false;
        if (!padded && !(repack_env && atoi(repack_env) == 0)) {
            const int rc = gemm_try_repacked(d, s, &done);
            if (done || rc) return rc;
        }
    }
    GemmPlan plan = gemm_fused_plan(d, padded);
    static const char* trace_env = getenv("NZHIP_TRACE");               // 1: one line per product on stderr (debugging only)
    if (trace_env && atoi(trace_env))
        fprintf(stderr, "nzhip_gemm %ld x %ld x %ld batch %ld x %ld%s: fused kernel, %d^2 tiles, %ld chunk(s) of %ld, model %.1f us\n",
                (long)d.M, (long)d.K, (long)d.N, (long)d.batch_n, (long)d.batch_c, padded ? " (padded copies)" : "", plan.tile,
                (long)plan.parts, (long)plan.Kc, plan.cost_us);
    static const char* sk_env = getenv("NZHIP_SPLITK");                  // benchmarking only: number of chunks
    if (sk_env && atoi(sk_env) >= 1 && d.batch_c == 1 && d.batch_n <= 65535) {
        const int64_t S = atoi(sk_env);
        plan.Kc = ((d.K + S - 1) / S + 31) / 32 * 32;
        plan.parts = (d.K + plan.Kc - 1) / plan.Kc;
    }
    if (plan.parts >= 2) {
        const int parts = (int)plan.parts;
        const int64_t Kc = plan.Kc;
        float* P = nullptr;
        if (int rc = workspace_alloc(reinterpret_cast<void**>(&P), (size_t)d.batch_n * parts * d.M * d.N * sizeof(float), s))
            return rc;
        nzhip_gemm_desc g = d;
        g.C = P; g.ldc = d.N; g.K = Kc;
        g.batch_c = parts;
        g.c_stride_n = (int64_t)parts * d.M * d.N;
        g.a_stride_c = d.a_layout == NZHIP_LAYOUT_ROW ? Kc : Kc * d.lda;   // next chunk of A / B
        g.b_stride_c = d.b_layout == NZHIP_LAYOUT_ROW ? Kc * d.ldb : Kc;
        g.c_stride_c = d.M * d.N;
        g.bias = nullptr; g.activation = NZHIP_ACT_NONE;
        int rc = gemm_mfma_dispatch(g, s, plan.tile, d.K, padded);
        if (rc == NZHIP_OK) {
            if (parts >= 64 && d.M * d.N <= 4096) {                     // a handful of outputs: one wave each
                const long groups = (d.M * d.N + 3) / 4;
                hipLaunchKernelGGL(splitk_reduce_wave_kernel, dim3((unsigned)groups, (unsigned)d.batch_n), dim3(256), 0, s, d, P, parts);
            } else if (parts > 16 || d.M * d.N < (1 << 18)) {           // few outputs: spread each over eight lanes
                const long groups = (d.M * d.N + 31) / 32;               // 32 outputs x 8 chunk lanes per workgroup
                hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)groups, (unsigned)d.batch_n), dim3(256), 0, s, d, P, parts);
            } else {
                const long groups = (d.M * d.N + 255) / 256;
                hipLaunchKernelGGL(splitk_reduce_wide_kernel, dim3((unsigned)groups, (unsigned)d.batch_n), dim3(256), 0, s, d, P, parts);
            }
            rc = check_launch("splitk_reduce_kernel");
        }
        const int rc2 = workspace_free(P, s);
        return rc ? rc : rc2;
    }
    return gemm_mfma_dispatch(d, s, 0, 0, padded);
}

extern "C" {

/* Test hook: pick the kernel instead of letting the shape decide. tile 64 / 128 / 256: the fused
 * convert-on-load kernel with that square tile; tile 16 / 18 / 12: the two-pass fp16 route with
 * 256x256 tiles and 4 waves / 256x256 tiles and 8 waves / 128x256 tiles, 16x16x32 MFMAs;
 * tile 316 / 318 / 312: the same three with 32x32x16 MFMAs. */
int nzhip_gemm_force_tile(const nzhip_gemm_desc* desc, int tile, void* stream) {
    if (!desc) return set_error(NZHIP_E_INVALID, "nzhip_gemm: null descriptor");
    const int base = tile > 300 ? tile - 300 : tile;
    if (tile != 64 && tile != 128 && tile != 256 && tile != 28 && base != 16 && base != 18 && base != 12)
        return set_error(NZHIP_E_INVALID, "nzhip_gemm_force_tile: tile must be 64, 128, 256, 16, 18, 12, 28, 316, 318 or 312");
    if (int rc = validate_gemm(*desc)) return rc;
    if (desc->M == 0 || desc->N == 0 || desc->K == 0) return nzhip_gemm(desc, stream);
    const int mfma = tile > 300 ? 32 : 16;
    if (tile == 28) {
        if (!gemm_h16_coop_applicable(*desc))
            return set_error(NZHIP_E_UNSUPPORTED, "nzhip_gemm_force_tile: the single-kernel route needs one product of whole 4096 x 4096 x 1024 blocks (and is off after a time-out)");
        return gemm_h16_coop_dispatch(*desc, as_stream(stream));
    }
    if (base == 16) return gemm_h16_dispatch(*desc, as_stream(stream), 4, mfma);
    if (base == 18) return gemm_h16_dispatch(*desc, as_stream(stream), 8, mfma);
    if (base == 12) return gemm_h16_dispatch(*desc, as_stream(stream), 2, mfma);
    return gemm_mfma_dispatch(*desc, as_stream(stream), tile);
}

int nzhip_gemm_coop_timeouts(unsigned* count) {
    if (!count) return set_error(NZHIP_E_INVALID, "nzhip_gemm_coop_timeouts: null pointer");
    return gemm_h16_coop_timeouts(count);
}

int nzhip_gemm_coop_reset(unsigned inject) { return gemm_h16_coop_reset(inject); }

int nzhip_gemm_coop_test_mode(unsigned spin_limit, int mute) {
    gemm_h16_coop_test_mode(spin_limit, mute);
    return NZHIP_OK;
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
    if (stride == 1 && K_h <= (size_t)I2C_MAXK && K_w <= (size_t)I2C_MAXK && (C * K_h * K_w) % 4 == 0 &&
        (I2C_CH * K_h * K_w) % 4 == 0 && aligned16(out)) {
        const size_t segs = (W_out + I2C_PX - 1) / I2C_PX, chunks = (C + I2C_CH - 1) / I2C_CH;
        // narrow images: as many whole rows per workgroup as make up 64 pixels and fit the staging space
        size_t rpw = 1;
        if (segs == 1) {
            rpw = I2C_PX / W_out;
            if (rpw > H_out) rpw = H_out;
            while (rpw > 1 && I2C_CH * (rpw + K_h - 1) * (W_out + K_w - 1) > (size_t)I2C_LDS) rpw--;
            if (rpw < 1) rpw = 1;
        }
        const size_t hblocks = (H_out + rpw - 1) / rpw;
        if (segs * hblocks <= 0x7fffffffull && chunks <= 65535) {
            dim3 grid((unsigned)(segs * hblocks), (unsigned)chunks, (unsigned)batch);
            auto kfn = (K_h == 3 && K_w == 3)   ? im2col_rows_kernel<3, 3>
                       : (K_h == 1 && K_w == 1) ? im2col_rows_kernel<1, 1>
                       : (K_h == 5 && K_w == 5) ? im2col_rows_kernel<5, 5>
                                                : im2col_rows_kernel<0, 0>;
            hipLaunchKernelGGL(kfn, grid, dim3(256), 0, as_stream(stream), out, in, (int)H_out, (int)W_out, (int)C, (int)K_h,
                               (int)K_w, (int)pad, (int)H_in, (int)W_in, (int)segs, (int)rpw);
            return check_launch("im2col_rows_kernel");
        }
    }
    if ((C * K_h * K_w) % 4 == 0 && aligned16(out)) {
        dim3 grid((unsigned)((per / 4 + 255) / 256), (unsigned)batch);
        hipLaunchKernelGGL(im2col_vec4_kernel, grid, dim3(256), 0, as_stream(stream), out, in, (int)H_out, (int)W_out,
                           (int)C, (int)K_h, (int)K_w, (int)stride, (int)pad, (int)H_in, (int)W_in);
        return check_launch("im2col_vec4_kernel");
    }
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
    if (C_out == 1 || HW == 1) {                                 // the transpose of a vector is a copy
        if (out == in) return NZHIP_OK;
        hipError_t e = hipMemcpyAsync(out, in, batches * HW * C_out * sizeof(float), hipMemcpyDeviceToDevice, as_stream(stream));
        return e == hipSuccess ? NZHIP_OK : set_hip_error(e, "hipMemcpyAsync (col2im of one channel)");
    }
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

int nzhip_fill(float* data, float value, size_t n, void* stream) {
    if (!data && n) return set_error(NZHIP_E_INVALID, "nzhip_fill: null pointer");
    if (n == 0) return NZHIP_OK;
    const int vec = aligned16(data);
    const size_t threads = vec ? (n + 3) / 4 : n;
    if ((threads + 255) / 256 > 0x7fffffffull) return set_error(NZHIP_E_UNSUPPORTED, "nzhip_fill: more than 2^39 elements");
    hipLaunchKernelGGL(fill_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, as_stream(stream), data, value, (long)n, vec);
    return check_launch("fill_kernel");
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

// ---- backward of the path ---------------------------------------------------------------------
namespace {

struct BwdOperand {
    const float* p;
    int layout;
    int64_t ld;
    int64_t sn, sc;                                        // batch strides, 0 = broadcast
};

// For every (i, j) of a bn x bc batch:  C[i*c_sn + j*c_sc] += f16(A_ij)[M,K] * f16(B_ij)[K,N].
// A batch stride of 0 on C makes that batch dimension a reduction (CuttingAndCompress,
// src/OperationKernels.cu:873-883, adds every member onto the same matrix). "+=" is the GEMM's bias
// operand pointed at C itself: every element is read and then written by the same lane.
// Reductions are folded into the contraction (K' = members x K, one launch) when both operands are
// laid out so that the member index continues the k index; otherwise the members are added one
// launch after the other, which fixes the summation order.
static int accumulate_products(float* C, int64_t ldc, int64_t c_sn, int64_t c_sc, BwdOperand A, BwdOperand B, int64_t M,
                        int64_t N, int64_t K, int64_t bn, int64_t bc, void* stream) {
    if (bn == 0 || bc == 0 || M == 0 || N == 0) return NZHIP_OK;
    auto launch = [&](const float* a, const float* b, float* c, int64_t k, int la, int64_t lda, int lb, int64_t ldb,
                      int64_t nb_n, int64_t nb_c, int64_t csn, int64_t csc) {
        nzhip_gemm_desc g = {};
        g.A = a; g.B = b; g.C = c;
        g.M = M; g.N = N; g.K = k;
        g.lda = lda; g.ldb = ldb; g.ldc = ldc;
        g.a_layout = la; g.b_layout = lb;
        g.batch_n = nb_n; g.batch_c = nb_c;
        g.a_stride_n = A.sn; g.a_stride_c = A.sc;
        g.b_stride_n = B.sn; g.b_stride_c = B.sc;
        g.c_stride_n = csn; g.c_stride_c = csc;
        g.bias = c;
        g.bias_stride_row = ldc; g.bias_stride_col = 1;
        g.bias_stride_n = csn; g.bias_stride_c = csc;
        return nzhip_gemm(&g, stream);
    };
    const bool red_n = c_sn == 0 && bn > 1, red_c = c_sc == 0 && bc > 1;
    // distance between consecutive batch members of an operand, if it is the same for all of them
    auto spacing = [&](int64_t sn, int64_t sc, int64_t& s) {
        if (bc == 1) { s = sn; return true; }
        if (bn == 1) { s = sc; return true; }
        s = sc;
        return sn == bc * sc;
    };
    if (!red_n && !red_c && bn * bc > 1 && K > 0) {
        // One shared matrix against a batch of vectors is a single GEMM whose rows are the members
        // (the shared operand is then read once instead of once per member).
        const int64_t T = bn * bc;
        int64_t sc_ = 0, sa = 0, sb = 0;
        const bool uc = spacing(c_sn, c_sc, sc_), ua = spacing(A.sn, A.sc, sa), ub = spacing(B.sn, B.sc, sb);
        const bool a_shared = A.sn == 0 && A.sc == 0, b_shared = B.sn == 0 && B.sc == 0;
        if (N == 1 && a_shared && uc && ub && ldc == 1 && sc_ >= M && sb >= K && (B.layout == NZHIP_LAYOUT_TRANS || B.ld == 1)) {
            // C_t[M,1] = A[M,K] * B_t[K,1]   ->   Cmat[T,M] = Bmat[T,K] * A^T
            nzhip_gemm_desc g = {};
            g.A = B.p; g.B = A.p; g.C = C;
            g.M = T; g.N = M; g.K = K;
            g.lda = sb; g.ldb = A.ld; g.ldc = sc_;
            g.a_layout = NZHIP_LAYOUT_ROW;
            g.b_layout = A.layout == NZHIP_LAYOUT_ROW ? NZHIP_LAYOUT_TRANS : NZHIP_LAYOUT_ROW;
            g.batch_n = g.batch_c = 1;
            g.bias = C; g.bias_stride_row = sc_; g.bias_stride_col = 1;
            return nzhip_gemm(&g, stream);
        }
        if (M == 1 && b_shared && uc && ua && sc_ >= N && sa >= K && (A.layout == NZHIP_LAYOUT_ROW || A.ld == 1)) {
            // C_t[1,N] = A_t[1,K] * B[K,N]   ->   Cmat[T,N] = Amat[T,K] * B
            nzhip_gemm_desc g = {};
            g.A = A.p; g.B = B.p; g.C = C;
            g.M = T; g.N = N; g.K = K;
            g.lda = sa; g.ldb = B.ld; g.ldc = sc_;
            g.a_layout = NZHIP_LAYOUT_ROW; g.b_layout = B.layout;
            g.batch_n = g.batch_c = 1;
            g.bias = C; g.bias_stride_row = sc_; g.bias_stride_col = 1;
            return nzhip_gemm(&g, stream);
        }
    }
    if (!red_n && !red_c) {
        if (bn * bc <= 65535) return launch(A.p, B.p, C, K, A.layout, A.ld, B.layout, B.ld, bn, bc, c_sn, c_sc);
        for (int64_t i = 0; i < bn; i++)
            for (int64_t j0 = 0; j0 < bc; j0 += 65535) {
                const int64_t cnt = bc - j0 < 65535 ? bc - j0 : 65535;
                if (int rc = launch(A.p + i * A.sn + j0 * A.sc, B.p + i * B.sn + j0 * B.sc, C + i * c_sn + j0 * c_sc, K,
                                    A.layout, A.ld, B.layout, B.ld, 1, cnt, 0, c_sc))
                    return rc;
            }
        return NZHIP_OK;
    }
    // every member reduces into one matrix and the members are evenly spaced: fold them into K
    const bool all = (red_n || bn == 1) && (red_c || bc == 1);
    if (all && K > 0) {
        const int64_t T = bn * bc;
        int64_t sa = 0, sb = 0;
        const bool ua = spacing(A.sn, A.sc, sa), ub = spacing(B.sn, B.sc, sb);
        int la = -1, lb = -1;
        int64_t lda = 0, ldb = 0;
        if (ua && A.layout == NZHIP_LAYOUT_TRANS && sa == K * A.ld) { la = NZHIP_LAYOUT_TRANS; lda = A.ld; }
        else if (ua && K == 1 && sa >= M && (A.layout == NZHIP_LAYOUT_TRANS || A.ld == 1)) { la = NZHIP_LAYOUT_TRANS; lda = sa; }
        if (ub && B.layout == NZHIP_LAYOUT_ROW && sb == K * B.ld) { lb = NZHIP_LAYOUT_ROW; ldb = B.ld; }
        else if (ub && K == 1 && sb >= N && (B.layout == NZHIP_LAYOUT_ROW || B.ld == 1)) { lb = NZHIP_LAYOUT_ROW; ldb = sb; }
        if (la >= 0 && lb >= 0 && T * K <= 0x3fffffff) {
            BwdOperand a1 = A, b1 = B;
            A.sn = A.sc = B.sn = B.sc = 0;                       // one member left
            const int rc = launch(a1.p, b1.p, C, T * K, la, lda, lb, ldb, 1, 1, 0, 0);
            A = a1; B = b1;
            return rc;
        }
    }
    // members one after the other; a dimension that does not reduce stays a batch of the launch
    for (int64_t i = 0; i < (red_n ? bn : 1); i++)
        for (int64_t j = 0; j < (red_c ? bc : 1); j++) {
            const int64_t nb_n = red_n ? 1 : bn, nb_c = red_c ? 1 : bc;
            if (nb_n * nb_c > 65535) return set_error(NZHIP_E_UNSUPPORTED, "gemm backward: more than 65535 batch members");
            if (int rc = launch(A.p + i * A.sn + j * A.sc, B.p + i * B.sn + j * B.sc, C, K, A.layout, A.ld, B.layout,
                                B.ld, nb_n, nb_c, c_sn, c_sc))
                return rc;
        }
    return NZHIP_OK;
}

inline int64_t bstride_n(const size_t s[4]) { return s[0] > 1 ? (int64_t)(s[1] * s[2] * s[3]) : 0; }
inline int64_t bstride_c(const size_t s[4]) { return s[1] > 1 ? (int64_t)(s[2] * s[3]) : 0; }

}  // namespace

int nzhip_gemm_backward(const float* A, const float* B, float* C, const size_t sA[4], const size_t sB[4],
                        const size_t sC[4], void* stream) {
    if (!A || !B || !C || !sA || !sB || !sC) return set_error(NZHIP_E_INVALID, "nzhip_gemm_backward: null argument");
    const int64_t M = (int64_t)sA[2], N = (int64_t)sB[3], K = (int64_t)sA[3];      // src/OperationKernels.cu:1032-1034
    const int64_t bn = (int64_t)(sA[0] > sB[0] ? sA[0] : sB[0]), bc = (int64_t)(sA[1] > sB[1] ? sA[1] : sB[1]);
    BwdOperand a = {A, NZHIP_LAYOUT_ROW, K, bstride_n(sA), bstride_c(sA)};
    BwdOperand b = {B, NZHIP_LAYOUT_ROW, N, bstride_n(sB), bstride_c(sB)};
    return accumulate_products(C, N, bstride_n(sC), bstride_c(sC), a, b, M, N, K, bn, bc, stream);   // :1116-1124
}

int nzhip_matmul_backward(float* dA, float* dB, const float* A, const float* B, const float* dC, const size_t sA[4],
                          const size_t sB[4], const size_t sC[4], void* stream) {
    if (!dC || !sA || !sB || !sC || (dA && !B) || (dB && !A))
        return set_error(NZHIP_E_INVALID, "nzhip_matmul_backward: null argument");
    const int64_t M = (int64_t)sA[2], K = (int64_t)sA[3], N = (int64_t)sB[3];
    if ((int64_t)sB[2] != K || (int64_t)sC[2] != M || (int64_t)sC[3] != N)
        return set_error(NZHIP_E_SHAPE, "nzhip_matmul_backward: shapes do not describe C = A * B");
    const int64_t bn = (int64_t)sC[0], bc = (int64_t)sC[1];
    const BwdOperand g = {dC, NZHIP_LAYOUT_ROW, N, (int64_t)(sC[1] * sC[2] * sC[3]), (int64_t)(sC[2] * sC[3])};
    if (dA) {                                              // dA += dC * B^T   (src/Nodes.cu:171-175)
        const BwdOperand bt = {B, NZHIP_LAYOUT_TRANS, N, bstride_n(sB), bstride_c(sB)};
        if (int rc = accumulate_products(dA, K, bstride_n(sA), bstride_c(sA), g, bt, M, K, N, bn, bc, stream)) return rc;
    }
    if (dB) {                                              // dB += A^T * dC   (src/Nodes.cu:177-181)
        const BwdOperand at = {A, NZHIP_LAYOUT_TRANS, K, bstride_n(sA), bstride_c(sA)};
        if (int rc = accumulate_products(dB, N, bstride_n(sB), bstride_c(sB), at, g, K, N, M, bn, bc, stream)) return rc;
    }
    return NZHIP_OK;
}

int nzhip_relu_backward(float* dx, const float* x, const float* dy, size_t n, void* stream) {
    if ((!dx || !x || !dy) && n) return set_error(NZHIP_E_INVALID, "nzhip_relu_backward: null pointer");
    if (n == 0) return NZHIP_OK;
    const int vec = aligned16(dx) && aligned16(x) && aligned16(dy);
    const size_t threads = vec ? (n + 3) / 4 : n;
    hipLaunchKernelGGL(relu_backward_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, as_stream(stream),
                       dx, x, dy, (long)n, vec);
    return check_launch("relu_backward_kernel");
}

int nzhip_add_backward(float* din, const float* dout, const size_t sIn[4], const size_t sOut[4], void* stream) {
    if (!din || !dout || !sIn || !sOut) return set_error(NZHIP_E_INVALID, "nzhip_add_backward: null argument");
    if (sIn[2] != sOut[2] || sIn[3] != sOut[3] || (sIn[0] != sOut[0] && sIn[0] != 1) || (sIn[1] != sOut[1] && sIn[1] != 1))
        return set_error(NZHIP_E_SHAPE, "Shapes are not broadcast compatible.");
    const size_t hw = sOut[2] * sOut[3], total = sOut[0] * sOut[1] * hw;
    if (total == 0) return NZHIP_OK;
    if (sIn[0] == sOut[0] && sIn[1] == sOut[1]) {          // src/Nodes.cu:101-105: plain copy
        hipError_t e = hipMemcpyAsync(din, dout, total * sizeof(float), hipMemcpyDeviceToDevice, as_stream(stream));
        return e == hipSuccess ? NZHIP_OK : set_hip_error(e, "hipMemcpyAsync(add backward)");
    }
    if (sIn[0] * sIn[1] > 65535 || sOut[0] > 0x7fffffff || sOut[1] > 0x7fffffff)
        return set_error(NZHIP_E_UNSUPPORTED, "nzhip_add_backward: more than 65535 (n,c) planes");
    dim3 grid((unsigned)((hw + 255) / 256), (unsigned)(sIn[0] * sIn[1]));
    const size_t members = (sIn[0] > 1 ? 1 : sOut[0]) * (sIn[1] > 1 ? 1 : sOut[1]);
    if (members >= (size_t)GRAD_CHUNK_MIN) {
        // enough chunks to put every CU to work, at least 16 members each
        const size_t threads = hw * sIn[0] * sIn[1];
        size_t chunks = ((size_t)device_cu_count() * 1024 + threads - 1) / threads;
        if (chunks > members / 16) chunks = members / 16;
        if (chunks > 1024) chunks = 1024;
        if (chunks >= 2) {
            const int chunk = (int)((members + chunks - 1) / chunks);
            chunks = (members + chunk - 1) / chunk;
            float* partial = nullptr;
            hipStream_t s = as_stream(stream);
            if (int rc = workspace_alloc(reinterpret_cast<void**>(&partial), chunks * threads * sizeof(float), s)) return rc;
            hipLaunchKernelGGL(grad_partial_kernel, dim3(grid.x, grid.y, (unsigned)chunks), dim3(256), 0, s, partial, dout, (long)hw,
                               (int)sIn[0], (int)sIn[1], (int)sOut[0], (int)sOut[1], chunk);
            int rc = check_launch("grad_partial_kernel");
            if (rc == NZHIP_OK) {
                hipLaunchKernelGGL(grad_partial_sum_kernel, grid, dim3(256), 0, s, din, partial, (long)hw, (int)chunks);
                rc = check_launch("grad_partial_sum_kernel");
            }
            const int rc2 = workspace_free(partial, s);
            return rc ? rc : rc2;
        }
    }
    hipLaunchKernelGGL(grad_reduce_kernel, grid, dim3(256), 0, as_stream(stream), din, dout, (long)hw, (int)sIn[0],
                       (int)sIn[1], (int)sOut[0], (int)sOut[1]);
    return check_launch("grad_reduce_kernel");
}

int nzhip_im2col_backward(float* dx, const float* dcol, size_t H_out, size_t W_out, size_t C, size_t K_h, size_t K_w,
                          size_t stride, size_t pad, size_t H_in, size_t W_in, size_t batch, void* stream) {
    if (!dx || !dcol) return set_error(NZHIP_E_INVALID, "nzhip_im2col_backward: null pointer");
    if (stride == 0 || K_h == 0 || K_w == 0)
        return set_error(NZHIP_E_INVALID, "nzhip_im2col_backward: zero stride or kernel extent");
    const size_t per = C * H_in * W_in;
    if (per == 0 || batch == 0 || H_out == 0 || W_out == 0) return NZHIP_OK;
    if (per > 0x7fffffffull * 256 || batch > 65535 || H_in > 0x3fffffff || W_in > 0x3fffffff || pad > 0x3fffffff ||
        H_out * W_out * C * K_h * K_w > 0x7fffffffffffull)
        return set_error(NZHIP_E_UNSUPPORTED, "nzhip_im2col_backward: extent too large");
    dim3 grid((unsigned)((per + 255) / 256), (unsigned)batch);
    hipLaunchKernelGGL(im2col_backward_kernel, grid, dim3(256), 0, as_stream(stream), dx, dcol, (int)H_out, (int)W_out,
                       (int)C, (int)K_h, (int)K_w, (int)stride, (int)pad, (int)H_in, (int)W_in);
    return check_launch("im2col_backward_kernel");
}

int nzhip_col2im_backward(float* dcol, const float* dy, size_t H_out, size_t W_out, size_t C_out, size_t batches,
                          void* stream) {
    if (!dcol || !dy) return set_error(NZHIP_E_INVALID, "nzhip_col2im_backward: null pointer");
    const size_t HW = H_out * W_out;
    if (HW == 0 || C_out == 0 || batches == 0) return NZHIP_OK;
    if (C_out > 0x7fffffff || (HW + 31) / 32 > 65535 || batches > 65535)
        return set_error(NZHIP_E_UNSUPPORTED, "nzhip_col2im_backward: extent too large");
    if (C_out == 1 || HW == 1) {                                 // the transpose of a vector is a copy
        if (dcol == dy) return NZHIP_OK;
        hipError_t e = hipMemcpyAsync(dcol, dy, batches * HW * C_out * sizeof(float), hipMemcpyDeviceToDevice, as_stream(stream));
        return e == hipSuccess ? NZHIP_OK : set_hip_error(e, "hipMemcpyAsync (col2im gradient of one channel)");
    }
    // the inverse transpose of col2im: [C_out, HW] -> [HW, C_out] per image
    dim3 grid((unsigned)((C_out + 31) / 32), (unsigned)((HW + 31) / 32), (unsigned)batches);
    hipLaunchKernelGGL(col2im_kernel, grid, dim3(256), 0, as_stream(stream), dcol, dy, (int)C_out, (int)HW);
    return check_launch("col2im_kernel (backward)");
}

}  // extern "C"
