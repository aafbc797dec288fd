// fp32-exact pieces next to the fp16 path: the matmul behind Tensor::operator* (no rounding of the
// operands, fp32 FMA accumulation in ascending k, reference: GeneralMatrixMulKernel,
// src/OperationKernels.cu:65-101) and the optimizer steps that close a training iteration
// (StochasticGradientDescentKernel :634-640, AdamKernel :753-766), plus the softmax forward and its
// Jacobian, whose product with the incoming gradient is one more call of the fp16 GEMM entry
// (SoftmaxNode::backward, src/Nodes.cu:538-548).
#include <hip/hip_runtime.h>

#include "nzhip_internal.h"

namespace nzhip {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));

static inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }
static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

static int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? NZHIP_OK : set_hip_error(e, what);
}

// ---- fp32 matmul --------------------------------------------------------------------------------
// 128 x 128 output tile per workgroup, four waves of 64 x 64 (2 x 2 blocks of v_mfma_f32_32x32x2_f32),
// k in steps of 16 through LDS (A stored k-major so that both fragment reads are 32 adjacent
// floats). The fp32 MFMA adds its two products to the accumulator one after the other, each as a
// fused multiply-add, in ascending k (checked on the device against a scalar chain over operands
// of widely different magnitudes: 1024 of 1024 outputs identical), so every output is the chain
// `sum = fma(a[k], b[k], sum)` of the CPU restatement, bit for bit; the tests hold it to that.
struct F32Args {
    const float* A;
    const float* B;
    float* C;
    int M, N, K;
    long a_sn, a_sc, b_sn, b_sc, c_sn, c_sc;
    int batch_c;
    int vec_a, vec_b;
};

constexpr int F32_BM = 128, F32_BN = 128, F32_BK = 16;

__global__ __launch_bounds__(256) void matmul_f32_kernel(const F32Args p) {
    __shared__ __attribute__((aligned(16))) float As[2][F32_BK][F32_BM + 4];   // [k][m]
    __shared__ __attribute__((aligned(16))) float Bs[2][F32_BK][F32_BN + 4];   // [k][n]
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * F32_BM, n0 = blockIdx.x * F32_BN;
    const int bi = blockIdx.z / p.batch_c, bj = blockIdx.z % p.batch_c;
    const float* __restrict__ A = p.A + bi * p.a_sn + bj * p.a_sc;
    const float* __restrict__ B = p.B + bi * p.b_sn + bj * p.b_sc;
    float* __restrict__ C = p.C + bi * p.c_sn + bj * p.c_sc;

    // staging: A tile 128 x 16 = 512 float4 along k (2 per thread); B tile 16 x 128 = 512 float4 along n
    floatx4 ra[2], rb[2];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int q = tid + h * 256;
            {   // A: row m = q / 4, k quad = q % 4
                const int m = m0 + (q >> 2), k = k0 + (q & 3) * 4;
                floatx4 v = {0.f, 0.f, 0.f, 0.f};
                if (m < p.M) {
                    const float* s = A + (long)m * p.K + k;
                    if (p.vec_a && k + 4 <= p.K) v = *reinterpret_cast<const floatx4*>(s);
                    else {
#pragma unroll
                        for (int e = 0; e < 4; e++) if (k + e < p.K) v[e] = s[e];
                    }
                }
                ra[h] = v;
            }
            {   // B: row k = q / 32, n quad = q % 32
                const int k = k0 + (q >> 5), n = n0 + (q & 31) * 4;
                floatx4 v = {0.f, 0.f, 0.f, 0.f};
                if (k < p.K) {
                    const float* s = B + (long)k * p.N + n;
                    if (p.vec_b && n + 4 <= p.N) v = *reinterpret_cast<const floatx4*>(s);
                    else {
#pragma unroll
                        for (int e = 0; e < 4; e++) if (n + e < p.N) v[e] = s[e];
                    }
                }
                rb[h] = v;
            }
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int q = tid + h * 256;
#pragma unroll
            for (int e = 0; e < 4; e++) As[buf][(q & 3) * 4 + e][q >> 2] = ra[h][e];
            *reinterpret_cast<floatx4*>(&Bs[buf][q >> 5][(q & 31) * 4]) = rb[h];
        }
    };

    const int lane = tid & 63, wave = tid >> 6, li = lane & 31, lh = lane >> 5;
    const int wm = wave >> 1, wn = wave & 1;
    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    const int nk = (p.K + F32_BK - 1) / F32_BK;
    fetch(0);
    stash(0);
    __syncthreads();
    for (int kt = 0; kt < nk; kt++) {
        const int buf = kt & 1;
        if (kt + 1 < nk) fetch((kt + 1) * F32_BK);
#pragma unroll
        for (int k = 0; k < F32_BK; k += 2) {
            // lane (li, lh) brings row / column li of its blocks at k + lh; zero rows past K add fma(0, 0, sum) = sum
            float a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; i++) a[i] = As[buf][k + lh][wm * 64 + i * 32 + li];
#pragma unroll
            for (int j = 0; j < 2; j++) b[j] = Bs[buf][k + lh][wn * 64 + j * 32 + li];
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk) stash(buf ^ 1);
        __syncthreads();
    }
    // accumulator register r of lane (li, lh): row (r / 4) * 8 + lh * 4 + r % 4, column li of the 32 x 32 block
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int m = m0 + wm * 64 + i * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
            if (m >= p.M) continue;
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int n = n0 + wn * 64 + j * 32 + li;
                if (n < p.N) C[(long)m * p.N + n] = acc[i][j][r];
            }
        }
}

// ---- optimizer steps ----------------------------------------------------------------------------
// One thread updates four adjacent elements (16-byte loads and stores) when the arrays are 16-byte
// aligned, one element otherwise; the last n % 4 elements go to the first threads of the last
// workgroup. The arithmetic per element is the same expression in every variant.
// The multiply-adds are spelled as FMAs (what a contracting compiler makes of `d -= lr * g` and of
// `m * beta1 + g * (1 - beta1)`), so that every variant of a kernel rounds the same way.
__device__ __forceinline__ float sgd_one(float d, float g, float lr) { return __builtin_fmaf(-lr, g, d); }

template <int VEC>
__global__ __launch_bounds__(256) void sgd_kernel(float* __restrict__ data, const float* __restrict__ grad, float lr,
                                                  long n) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if constexpr (VEC == 4) {
        const long n4 = n >> 2;
        if (i < n4) {
            floatx4 d = reinterpret_cast<const floatx4*>(data)[i];
            const floatx4 g = reinterpret_cast<const floatx4*>(grad)[i];
#pragma unroll
            for (int e = 0; e < 4; e++) d[e] = sgd_one(d[e], g[e], lr);
            reinterpret_cast<floatx4*>(data)[i] = d;
        }
        const long t = n4 * 4 + threadIdx.x;
        if (blockIdx.x == gridDim.x - 1 && t < n) data[t] = sgd_one(data[t], grad[t], lr);
    } else {
        if (i < n) data[i] = sgd_one(data[i], grad[i], lr);
    }
}

// bias corrections 1 - beta^t are computed once on the host (in fp32, like the kernel of the reference)
struct AdamArgs {
    float lr, beta1, beta2, eps, corr1, corr2;
};

__device__ __forceinline__ void adam_one(float& d, float& m, float& v, float g, const AdamArgs& a) {
    const float m_temp = __builtin_fmaf(m, a.beta1, g * (1 - a.beta1));
    const float v_temp = __builtin_fmaf(v, a.beta2, (g * g) * (1 - a.beta2));
    const float m_modified = m_temp / a.corr1;
    const float v_modified = v_temp / a.corr2;
    d -= a.lr * m_modified / (sqrtf(v_modified) + a.eps);
    m = m_temp;
    v = v_temp;
}

template <int VEC>
__global__ __launch_bounds__(256) void adam_kernel(float* __restrict__ data, float* __restrict__ m,
                                                   float* __restrict__ v, const float* __restrict__ grad,
                                                   const AdamArgs a, long n) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if constexpr (VEC == 4) {
        const long n4 = n >> 2;
        if (i < n4) {
            floatx4 d = reinterpret_cast<const floatx4*>(data)[i];
            floatx4 mm = reinterpret_cast<const floatx4*>(m)[i];
            floatx4 vv = reinterpret_cast<const floatx4*>(v)[i];
            const floatx4 g = reinterpret_cast<const floatx4*>(grad)[i];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                float de = d[e], me = mm[e], ve = vv[e];
                adam_one(de, me, ve, g[e], a);
                d[e] = de; mm[e] = me; vv[e] = ve;
            }
            reinterpret_cast<floatx4*>(data)[i] = d;
            reinterpret_cast<floatx4*>(m)[i] = mm;
            reinterpret_cast<floatx4*>(v)[i] = vv;
        }
        const long t = n4 * 4 + threadIdx.x;
        if (blockIdx.x == gridDim.x - 1 && t < n) adam_one(data[t], m[t], v[t], grad[t], a);
    } else {
        if (i < n) adam_one(data[i], m[i], v[i], grad[i], a);
    }
}

// ---- the same steps for several tensors in one launch ------------------------------------------
// A small network has a dozen parameter tensors of a few floats each: one launch per tensor is a dozen launch
// latencies for microseconds of work. Workgroups [first[k], first[k + 1]) belong to tensor k and do exactly what
// the one-tensor kernel does with them (same element arithmetic, same 16-byte / scalar choice per tensor).
constexpr int MANY_MAX = NZHIP_MANY_MAX;
struct ManyArgs {
    float* data[MANY_MAX];
    float* m[MANY_MAX];
    float* v[MANY_MAX];
    const float* grad[MANY_MAX];
    long n[MANY_MAX];
    unsigned first[MANY_MAX + 1];
    float corr1[MANY_MAX], corr2[MANY_MAX];
    unsigned vec_mask;
    int count;
    float lr, beta1, beta2, eps, value;
};

__device__ __forceinline__ int many_tensor_of(const ManyArgs& a, unsigned block) {
    int k = 0;
    while (k + 1 < a.count && block >= a.first[k + 1]) k++;     // (uniform)
    return k;
}

// MODE 0: fill with a.value; 1: SGD; 2: Adam
template <int MODE>
__global__ __launch_bounds__(256) void many_kernel(const ManyArgs a) {
    const int k = many_tensor_of(a, blockIdx.x);
    const unsigned blk = blockIdx.x - a.first[k], n_blk = a.first[k + 1] - a.first[k];
    float* data = a.data[k];
    const float* grad = a.grad[k];
    const long n = a.n[k];
    const long i = (long)blk * 256 + threadIdx.x;
    AdamArgs ad;
    ad.lr = a.lr; ad.beta1 = a.beta1; ad.beta2 = a.beta2; ad.eps = a.eps; ad.corr1 = a.corr1[k]; ad.corr2 = a.corr2[k];
    auto one = [&](const long e) {
        if (MODE == 0) data[e] = a.value;
        else if (MODE == 1) data[e] = sgd_one(data[e], grad[e], a.lr);
        else adam_one(data[e], a.m[k][e], a.v[k][e], grad[e], ad);
    };
    if (a.vec_mask >> k & 1) {
        const long n4 = n >> 2;
        if (i < n4) {
            if (MODE == 0) {
                const floatx4 f = {a.value, a.value, a.value, a.value};
                reinterpret_cast<floatx4*>(data)[i] = f;
            } else if (MODE == 1) {
                floatx4 d = reinterpret_cast<const floatx4*>(data)[i];
                const floatx4 g = reinterpret_cast<const floatx4*>(grad)[i];
#pragma unroll
                for (int e = 0; e < 4; e++) d[e] = sgd_one(d[e], g[e], a.lr);
                reinterpret_cast<floatx4*>(data)[i] = d;
            } else {
                floatx4 d = reinterpret_cast<const floatx4*>(data)[i];
                floatx4 mm = reinterpret_cast<const floatx4*>(a.m[k])[i];
                floatx4 vv = reinterpret_cast<const floatx4*>(a.v[k])[i];
                const floatx4 g = reinterpret_cast<const floatx4*>(grad)[i];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float de = d[e], me = mm[e], ve = vv[e];
                    adam_one(de, me, ve, g[e], ad);
                    d[e] = de; mm[e] = me; vv[e] = ve;
                }
                reinterpret_cast<floatx4*>(data)[i] = d;
                reinterpret_cast<floatx4*>(a.m[k])[i] = mm;
                reinterpret_cast<floatx4*>(a.v[k])[i] = vv;
            }
        }
        const long t = n4 * 4 + threadIdx.x;
        if (blk == n_blk - 1 && t < n) one(t);
    } else if (i < n) {
        one(i);
    }
}

// ---- softmax over one vector per (n, c) and its Jacobian ---------------------------------------
// One workgroup per vector: exp(x) summed in a fixed tree order (lane stride, wave shuffle, four
// waves), then every element divided by the sum. No maximum is subtracted, like the reference
// (SummationExpKernel / SoftmaxKernel, src/OperationKernels.cu:477-523).
__global__ __launch_bounds__(256) void softmax_kernel(float* __restrict__ out, const float* __restrict__ in, long len) {
    __shared__ float part[4];
    const float* x = in + (long)blockIdx.x * len;
    float* y = out + (long)blockIdx.x * len;
    float s = 0.f;
    for (long i = threadIdx.x; i < len; i += 256) s += __expf(x[i]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s += __shfl_down(s, off);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
    __syncthreads();
    const float total = (part[0] + part[1]) + (part[2] + part[3]);
    for (long i = threadIdx.x; i < len; i += 256) y[i] = __expf(x[i]) / total;
}

// SoftmaxJacobianKernel (:550-565): J[x][y] = s_x (1 - s_x) on the diagonal, -s_x s_y elsewhere.
__global__ __launch_bounds__(256) void softmax_jacobian_kernel(float* __restrict__ out, const float* __restrict__ in,
                                                               int n) {
    const long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= (long)n * n) return;
    const int r = (int)(t / n), c = (int)(t % n);
    const float* s = in + (long)blockIdx.y * n;
    out[(long)blockIdx.y * n * n + t] = r == c ? s[r] * (1 - s[r]) : -s[r] * s[c];
}

// SoftmaxNode::backward (src/Nodes.cu:538-548) without the n x n Jacobian in memory: output i is
//   sum_j fp16(J[i][j]) * fp16(dy[j]),  J[i][j] = s_i (1 - s_i) if i == j else -s_i s_j,
// the Jacobian entry computed in fp32 exactly as softmax_jacobian_kernel does, rounded to fp16 like an
// operand of the GEMM, multiplied with the rounded gradient (exact in fp32) and added in ascending j.
// The Jacobian is symmetric, so J x dy (column vectors) and dy x J (row vectors) are the same sums.
// One thread per output i; s and the rounded gradient pass through LDS in chunks of SB_CHUNK entries.
constexpr int SB_CHUNK = 1024;

// fp16(fp32(s_i * t)): two roundings, like a Jacobian stored in fp32 and then rounded as a GEMM operand.
// The empty asm keeps the compiler from folding the product and the conversion into one mixed-precision
// FMA, which rounds the exact product once and differs in the last fp16 bit now and then.
__device__ __forceinline__ float jacobian_entry_f16(float si, float t) {
    float p = si * t;
    asm volatile("" : "+v"(p));
    return (float)(_Float16)p;
}

__global__ __launch_bounds__(256) void softmax_backward_kernel(float* __restrict__ dx, const float* __restrict__ s,
                                                               const float* __restrict__ dy, int n) {
    __shared__ __attribute__((aligned(16))) float tj[SB_CHUNK];        // -s_j
    __shared__ __attribute__((aligned(16))) _Float16 gj[SB_CHUNK];     // fp16(dy_j)
    const float* sv = s + (long)blockIdx.y * n;
    const float* gv = dy + (long)blockIdx.y * n;
    const int i = blockIdx.x * 256 + threadIdx.x;
    const float si = i < n ? sv[i] : 0.f;
    const float diag = 1 - si;
    float acc = 0.f;
    for (int j0 = 0; j0 < n; j0 += SB_CHUNK) {
        const int cnt = min(SB_CHUNK, n - j0);
        __syncthreads();
        for (int q = threadIdx.x; q < cnt; q += 256) {
            tj[q] = -sv[j0 + q];
            gj[q] = (_Float16)gv[j0 + q];
        }
        __syncthreads();
        // the chunk holding this workgroup's own outputs (256 | SB_CHUNK) needs the diagonal term
        const bool own = (blockIdx.x * 256) / SB_CHUNK == j0 / SB_CHUNK;
        const int jd = own ? i - j0 : -1;
        int q = 0;
        for (; q + 8 <= cnt; q += 8) {
            const floatx4 ta = *reinterpret_cast<const floatx4*>(&tj[q]);
            const floatx4 tb = *reinterpret_cast<const floatx4*>(&tj[q + 4]);
            const halfx8 g8 = *reinterpret_cast<const halfx8*>(&gj[q]);
            if (own) {      // uniform over the workgroup
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const float t = q + e == jd ? diag : (e < 4 ? ta[e] : tb[e - 4]);
                    acc = __builtin_fmaf(jacobian_entry_f16(si, t), (float)g8[e], acc);
                }
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++)
                    acc = __builtin_fmaf(jacobian_entry_f16(si, e < 4 ? ta[e] : tb[e - 4]), (float)g8[e], acc);
            }
        }
        for (; q < cnt; q++) acc = __builtin_fmaf(jacobian_entry_f16(si, q == jd ? diag : tj[q]), (float)gj[q], acc);
    }
    if (i < n) dx[(long)blockIdx.y * n + i] = acc;
}

}  // namespace nzhip

using namespace nzhip;

// Launches many_kernel<MODE> over tensors [0, count) in groups of at most MANY_MAX
template <int MODE>
static int many_launch(const char* who, int count, float* const* data, float* const* m, float* const* v, const float* const* grad,
                       const size_t* n, const int* t, float lr, float beta1, float beta2, float eps, float value, void* stream) {
    if (count < 0) return set_error(NZHIP_E_INVALID, "%s: negative count", who);
    if (count && (!data || !n || (MODE >= 1 && !grad) || (MODE == 2 && (!m || !v || !t))))
        return set_error(NZHIP_E_INVALID, "%s: null pointer", who);
    for (int k = 0; k < count; k++) {
        if (n[k] && (!data[k] || (MODE >= 1 && !grad[k]) || (MODE == 2 && (!m[k] || !v[k]))))
            return set_error(NZHIP_E_INVALID, "%s: null pointer (tensor %d)", who, k);
        if (MODE == 2 && t[k] < 1) return set_error(NZHIP_E_INVALID, "%s: the step count starts at 1 (tensor %d)", who, k);
    }
    int k = 0;
    while (k < count) {
        ManyArgs a = {};
        a.lr = lr; a.beta1 = beta1; a.beta2 = beta2; a.eps = eps; a.value = value;
        unsigned long long blocks = 0;
        for (; k < count && a.count < MANY_MAX; k++) {
            if (n[k] == 0) continue;
            const int j = a.count;
            const bool vec = aligned16(data[k]) && (MODE < 1 || aligned16(grad[k])) && (MODE < 2 || (aligned16(m[k]) && aligned16(v[k]))) &&
                             n[k] >= 4;
            const unsigned long long nb = vec ? (n[k] / 4 + 255) / 256 : (n[k] + 255) / 256;
            if (blocks + nb > 0x7fffffffull) {
                if (a.count == 0) return set_error(NZHIP_E_UNSUPPORTED, "%s: more than 2^39 elements in one tensor", who);
                break;                                            // this tensor starts the next launch
            }
            a.data[j] = data[k];
            a.grad[j] = MODE >= 1 ? grad[k] : nullptr;
            a.m[j] = MODE == 2 ? m[k] : nullptr;
            a.v[j] = MODE == 2 ? v[k] : nullptr;
            a.n[j] = (long)n[k];
            if (MODE == 2) {
                a.corr1[j] = 1.0f - powf(beta1, (float)t[k]);
                a.corr2[j] = 1.0f - powf(beta2, (float)t[k]);
            }
            if (vec) a.vec_mask |= 1u << j;
            a.first[j] = (unsigned)blocks;
            blocks += nb;
            a.first[j + 1] = (unsigned)blocks;
            a.count++;
        }
        if (a.count == 0) continue;
        hipLaunchKernelGGL(many_kernel<MODE>, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), a);
        if (int rc = check_launch("many_kernel")) return rc;
    }
    return NZHIP_OK;
}

extern "C" {

int nzhip_matmul_f32(const float* A, const float* B, float* C, const size_t sA[4], const size_t sB[4],
                     const size_t sC[4], void* stream) {
    if (!A || !B || !C || !sA || !sB || !sC) return set_error(NZHIP_E_INVALID, "nzhip_matmul_f32: null argument");
    for (int i = 0; i < 2; i++)
        if (sA[i] != sB[i] && sA[i] != 1 && sB[i] != 1) return set_error(NZHIP_E_SHAPE, "Shapes are not broadcast compatible.");
    if (sA[3] != sB[2]) return set_error(NZHIP_E_SHAPE, "Shapes are not broadcast compatible.");
    const size_t M = sA[2], N = sB[3], K = sA[3];
    const size_t bn = sC[0], bc = sC[1];
    if (M == 0 || N == 0 || bn == 0 || bc == 0) return NZHIP_OK;
    if (M > 0x3fffffff || N > 0x3fffffff || K > 0x3fffffff || bn * bc > 65535 || (M + F32_BM - 1) / F32_BM > 65535)
        return set_error(NZHIP_E_UNSUPPORTED, "nzhip_matmul_f32: extent too large");
    F32Args a;
    a.A = A; a.B = B; a.C = C;
    a.M = (int)M; a.N = (int)N; a.K = (int)K;
    a.a_sn = sA[0] > 1 ? (long)(sA[1] * sA[2] * sA[3]) : 0;      // TensorOperations.cuh:1006-1014
    a.a_sc = sA[1] > 1 ? (long)(sA[2] * sA[3]) : 0;
    a.b_sn = sB[0] > 1 ? (long)(sB[1] * sB[2] * sB[3]) : 0;
    a.b_sc = sB[1] > 1 ? (long)(sB[2] * sB[3]) : 0;
    a.c_sn = (long)(sC[1] * sC[2] * sC[3]);
    a.c_sc = (long)(sC[2] * sC[3]);
    a.batch_c = (int)bc;
    a.vec_a = aligned16(A) && (K % 4 == 0);
    a.vec_b = aligned16(B) && (N % 4 == 0);
    dim3 grid((unsigned)((N + F32_BN - 1) / F32_BN), (unsigned)((M + F32_BM - 1) / F32_BM), (unsigned)(bn * bc));
    hipLaunchKernelGGL(matmul_f32_kernel, grid, dim3(256), 0, as_stream(stream), a);
    return check_launch("matmul_f32_kernel");
}

int nzhip_sgd_step(float* data, const float* grad, float lr, size_t n, void* stream) {
    if ((!data || !grad) && n) return set_error(NZHIP_E_INVALID, "nzhip_sgd_step: null pointer");
    if (n == 0) return NZHIP_OK;
    if (aligned16(data) && aligned16(grad) && n >= 4)
        hipLaunchKernelGGL(sgd_kernel<4>, dim3((unsigned)((n / 4 + 255) / 256)), dim3(256), 0, as_stream(stream), data, grad,
                           lr, (long)n);
    else
        hipLaunchKernelGGL(sgd_kernel<1>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, as_stream(stream), data, grad, lr,
                           (long)n);
    return check_launch("sgd_kernel");
}

int nzhip_adam_step(float* data, float* m, float* v, const float* grad, float lr, float beta1, float beta2, float eps,
                    int t, size_t n, void* stream) {
    if ((!data || !m || !v || !grad) && n) return set_error(NZHIP_E_INVALID, "nzhip_adam_step: null pointer");
    if (t < 1) return set_error(NZHIP_E_INVALID, "nzhip_adam_step: the step count starts at 1");
    if (n == 0) return NZHIP_OK;
    AdamArgs a;
    a.lr = lr; a.beta1 = beta1; a.beta2 = beta2; a.eps = eps;
    a.corr1 = 1.0f - powf(beta1, (float)t);
    a.corr2 = 1.0f - powf(beta2, (float)t);
    if (aligned16(data) && aligned16(m) && aligned16(v) && aligned16(grad) && n >= 4)
        hipLaunchKernelGGL(adam_kernel<4>, dim3((unsigned)((n / 4 + 255) / 256)), dim3(256), 0, as_stream(stream), data, m, v,
                           grad, a, (long)n);
    else
        hipLaunchKernelGGL(adam_kernel<1>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, as_stream(stream), data, m, v,
                           grad, a, (long)n);
    return check_launch("adam_kernel");
}

int nzhip_fill_many(int count, float* const* data, const size_t* n, float value, void* stream) {
    return many_launch<0>("nzhip_fill_many", count, data, nullptr, nullptr, nullptr, n, nullptr, 0.f, 0.f, 0.f, 0.f, value, stream);
}

int nzhip_sgd_step_many(int count, float* const* data, const float* const* grad, const size_t* n, float lr, void* stream) {
    return many_launch<1>("nzhip_sgd_step_many", count, data, nullptr, nullptr, grad, n, nullptr, lr, 0.f, 0.f, 0.f, 0.f, stream);
}

int nzhip_adam_step_many(int count, float* const* data, float* const* m, float* const* v, const float* const* grad, const size_t* n,
                         const int* t, float lr, float beta1, float beta2, float eps, void* stream) {
    return many_launch<2>("nzhip_adam_step_many", count, data, m, v, grad, n, t, lr, beta1, beta2, eps, 0.f, stream);
}

int nzhip_softmax(float* out, const float* in, size_t len, size_t batch, void* stream) {
    if ((!out || !in) && len * batch) return set_error(NZHIP_E_INVALID, "nzhip_softmax: null pointer");
    if (len == 0 || batch == 0) return NZHIP_OK;
    if (batch > 0x7fffffff) return set_error(NZHIP_E_UNSUPPORTED, "nzhip_softmax: too many vectors");
    hipLaunchKernelGGL(softmax_kernel, dim3((unsigned)batch), dim3(256), 0, as_stream(stream), out, in, (long)len);
    return check_launch("softmax_kernel");
}

int nzhip_softmax_jacobian(float* out, const float* in, size_t n, size_t batch, void* stream) {
    if ((!out || !in) && n * batch) return set_error(NZHIP_E_INVALID, "nzhip_softmax_jacobian: null pointer");
    if (n == 0 || batch == 0) return NZHIP_OK;
    if (n > 46340 || batch > 65535) return set_error(NZHIP_E_UNSUPPORTED, "nzhip_softmax_jacobian: extent too large");
    dim3 grid((unsigned)((n * n + 255) / 256), (unsigned)batch);
    hipLaunchKernelGGL(softmax_jacobian_kernel, grid, dim3(256), 0, as_stream(stream), out, in, (int)n);
    return check_launch("softmax_jacobian_kernel");
}

int nzhip_softmax_backward(float* dx, const float* s, const float* dy, size_t n, size_t batch, void* stream) {
    if ((!dx || !s || !dy) && n * batch) return set_error(NZHIP_E_INVALID, "nzhip_softmax_backward: null pointer");
    if (n == 0 || batch == 0) return NZHIP_OK;
    if (n > 0x3fffffff || batch > 65535) return set_error(NZHIP_E_UNSUPPORTED, "nzhip_softmax_backward: extent too large");
    dim3 grid((unsigned)((n + 255) / 256), (unsigned)batch);
    hipLaunchKernelGGL(softmax_backward_kernel, grid, dim3(256), 0, as_stream(stream), dx, s, dy, (int)n);
    return check_launch("softmax_backward_kernel");
}

}  // extern "C"
