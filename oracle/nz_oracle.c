/*
 * nz_oracle.c -- CPU restatement of NeuZephyr's tensor-core GEMM path.
 * TEST INFRASTRUCTURE ONLY (checker + timed CPU baseline); see nz_oracle.h.
 *
 * Build: oracle/Makefile (gcc -O3 -fopenmp, two ISA levels).
 */
#include "nz_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------- */
/* fp32 -> fp16 (IEEE binary16) round-to-nearest-even, in integer arithmetic. */
/* Restates __float2half as used by Padding (src/OperationKernels.cu:854).    */
/* ------------------------------------------------------------------------- */
uint16_t nzo_f32_to_f16_bits(float x) {
    uint32_t u;
    memcpy(&u, &x, 4);
    const uint32_t sign = (u >> 16) & 0x8000u;
    const uint32_t absu = u & 0x7fffffffu;
    if (absu >= 0x7f800000u) {                       /* inf / NaN */
        if (absu == 0x7f800000u) return (uint16_t)(sign | 0x7c00u);
        /* quiet NaN, keep top payload bits (what F16C and the GPU converters do) */
        return (uint16_t)(sign | 0x7e00u | ((absu >> 13) & 0x01ffu));
    }
    if (absu >= 0x477ff000u) {                       /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (absu >= 0x38800000u) {                       /* normal half range: >= 2^-14 */
        /* rebias exponent 127 -> 15, round mantissa 23 -> 10 bits (RNE) */
        const uint32_t v = absu - 0x38000000u;       /* exponent rebias */
        const uint32_t lsb = (v >> 13) & 1u;
        const uint32_t r = v + 0x0fffu + lsb;        /* carries into exponent correctly */
        return (uint16_t)(sign | (r >> 13));
    }
    if (absu < 0x33000000u) {                        /* < 2^-25: rounds to zero */
        return (uint16_t)sign;                       /* (exactly 2^-25 is a tie -> even = 0) */
    }
    /* subnormal half: value = m * 2^-24, m in [0,1024) */
    {
        const int e = (int)(absu >> 23);             /* biased fp32 exponent, 102..112 */
        const uint32_t man = (absu & 0x007fffffu) | 0x00800000u;   /* 24-bit significand */
        const int shift = 126 - e;                   /* bits dropped: 14..24 */
        const uint32_t q = man >> shift;
        const uint32_t rem = man & ((1u << shift) - 1u);
        const uint32_t half = 1u << (shift - 1);
        uint32_t m = q;
        if (rem > half || (rem == half && (q & 1u))) m++;
        return (uint16_t)(sign | m);                 /* m == 1024 becomes the smallest normal */
    }
}

float nzo_f16_bits_to_f32(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1fu;
    uint32_t m = h & 0x3ffu;
    uint32_t u;
    if (e == 0x1f) {
        u = sign | 0x7f800000u | (m << 13);
        if (m) u |= 0x00400000u;                     /* signalling NaNs are quieted, as VCVTPH2PS does */
    } else if (e != 0) {
        u = sign | ((e + 112u) << 23) | (m << 13);
    } else if (m == 0) {
        u = sign;
    } else {                                         /* subnormal: normalise */
        int sh = 0;
        while (!(m & 0x400u)) { m <<= 1; sh++; }
        m &= 0x3ffu;
        u = sign | ((uint32_t)(113 - sh) << 23) | (m << 13);
    }
    float f;
    memcpy(&f, &u, 4);
    return f;
}

float nzo_round_f16(float x) { return nzo_f16_bits_to_f32(nzo_f32_to_f16_bits(x)); }

void nzo_round_f16_array(float* dst, const float* src, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; i++) dst[i] = nzo_round_f16(src[i]);
}

/* ------------------------------------------------------------------------- */
/* GEMM: fp16-rounded operands held as fp32, fp32 accumulation, k ascending.  */
/* src/OperationKernels.cu:821-844 (the mma loop, :837-841) with the rounding */
/* of Padding (:846-860).  Products of two halfs are exact in fp32, so        */
/* mul+add and fma agree; only the order of the k sum is a free choice.       */
/* ------------------------------------------------------------------------- */

/* Pack rounded copies so the inner loops stream contiguous memory:
 * Ar[M][K] row-major, Br[K][N] row-major (transposing when trans_b). */
static float* round_pack_a(const float* A, size_t row0, size_t M, size_t K, size_t lda) {
    float* Ar = (float*)malloc(sizeof(float) * (M ? M : 1) * (K ? K : 1));
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < M; i++)
        for (size_t k = 0; k < K; k++) Ar[i * K + k] = nzo_round_f16(A[(row0 + i) * lda + k]);
    return Ar;
}

static float* round_pack_b(const float* B, size_t K, size_t N, size_t ldb, int trans_b) {
    float* Br = (float*)malloc(sizeof(float) * (K ? K : 1) * (N ? N : 1));
    if (!trans_b) {
#pragma omp parallel for schedule(static)
        for (size_t k = 0; k < K; k++)
            for (size_t n = 0; n < N; n++) Br[k * N + n] = nzo_round_f16(B[k * ldb + n]);
    } else {
#pragma omp parallel for schedule(static)
        for (size_t n = 0; n < N; n++)
            for (size_t k = 0; k < K; k++) Br[k * N + n] = nzo_round_f16(B[n * ldb + k]);
    }
    return Br;
}

/* Cache/register blocking. Per output element the k sum stays strictly ascending:
 * k blocks are visited in ascending order and the partial sum is carried in C. */
#define NZO_KB 256   /* k block: a Br panel of KB x NB floats stays in L2 */
#define NZO_NB 512   /* n block */
#define NZO_MR 4     /* register tile rows */
#define NZO_NR 64    /* register tile cols (4 zmm / 8 ymm of floats) */

#define NZO_DEFINE_GEMM_ROWS(NAME, ACC_T)                                                          \
    static void NAME(const float* Ar, const float* Br, ACC_T* C, size_t M, size_t N, size_t K,     \
                     size_t ldc) {                                                                 \
        const size_t MBLK = 32;                                                                    \
        const size_t nmb = (M + MBLK - 1) / MBLK;                                                  \
        const size_t nnb = (N + NZO_NB - 1) / NZO_NB;                                              \
        _Pragma("omp parallel for collapse(2) schedule(dynamic, 1)")                               \
        for (size_t mb = 0; mb < nmb; mb++) {                                                      \
            for (size_t nb = 0; nb < nnb; nb++) {                                                  \
                const size_t i0 = mb * MBLK, i1 = i0 + MBLK < M ? i0 + MBLK : M;                   \
                const size_t n0 = nb * NZO_NB, n1 = n0 + NZO_NB < N ? n0 + NZO_NB : N;             \
                for (size_t i = i0; i < i1; i++)                                                   \
                    for (size_t n = n0; n < n1; n++) C[i * ldc + n] = 0;                           \
                for (size_t k0 = 0; k0 < K; k0 += NZO_KB) {                                        \
                    const size_t k1 = k0 + NZO_KB < K ? k0 + NZO_KB : K;                           \
                    for (size_t i = i0; i < i1; i += NZO_MR) {                                     \
                        const size_t mr = i + NZO_MR <= i1 ? NZO_MR : i1 - i;                      \
                        for (size_t n = n0; n < n1; n += NZO_NR) {                                 \
                            const size_t nr = n + NZO_NR <= n1 ? NZO_NR : n1 - n;                  \
                            ACC_T acc[NZO_MR][NZO_NR];                                             \
                            if (mr == NZO_MR && nr == NZO_NR) {                                    \
                                for (int r = 0; r < NZO_MR; r++)                                   \
                                    for (int q = 0; q < NZO_NR; q++) acc[r][q] = C[(i + r) * ldc + n + q]; \
                                for (size_t k = k0; k < k1; k++) {                                 \
                                    const float* b = Br + k * N + n;                               \
                                    for (int r = 0; r < NZO_MR; r++) {                             \
                                        const ACC_T a = (ACC_T)Ar[(i + r) * K + k];                \
                                        _Pragma("omp simd")                                        \
                                        for (int q = 0; q < NZO_NR; q++) acc[r][q] += a * (ACC_T)b[q]; \
                                    }                                                              \
                                }                                                                  \
                                for (int r = 0; r < NZO_MR; r++)                                   \
                                    for (int q = 0; q < NZO_NR; q++) C[(i + r) * ldc + n + q] = acc[r][q]; \
                            } else {                                                               \
                                for (size_t r = 0; r < mr; r++)                                    \
                                    for (size_t q = 0; q < nr; q++) {                              \
                                        ACC_T s = C[(i + r) * ldc + n + q];                        \
                                        for (size_t k = k0; k < k1; k++)                           \
                                            s += (ACC_T)Ar[(i + r) * K + k] * (ACC_T)Br[k * N + n + q]; \
                                        C[(i + r) * ldc + n + q] = s;                              \
                                    }                                                              \
                            }                                                                      \
                        }                                                                          \
                    }                                                                              \
                }                                                                                  \
            }                                                                                      \
        }                                                                                          \
    }

NZO_DEFINE_GEMM_ROWS(gemm_rows_f32, float)
NZO_DEFINE_GEMM_ROWS(gemm_rows_f64, double)

void nzo_gemm_f16in_f32acc(const float* A, const float* B, float* C, size_t M, size_t N, size_t K,
                           size_t lda, size_t ldb, size_t ldc, int trans_b) {
    float* Ar = round_pack_a(A, 0, M, K, lda);
    float* Br = round_pack_b(B, K, N, ldb, trans_b);
    gemm_rows_f32(Ar, Br, C, M, N, K, ldc);
    free(Ar);
    free(Br);
}

void nzo_gemm_f16in_f64acc(const float* A, const float* B, double* C, size_t M, size_t N, size_t K,
                           size_t lda, size_t ldb, size_t ldc, int trans_b) {
    float* Ar = round_pack_a(A, 0, M, K, lda);
    float* Br = round_pack_b(B, K, N, ldb, trans_b);
    gemm_rows_f64(Ar, Br, C, M, N, K, ldc);
    free(Ar);
    free(Br);
}

void nzo_gemm_rows(const float* A, const float* B, float* C32, double* C64, size_t row0, size_t nrows,
                   size_t N, size_t K, size_t lda, size_t ldb, int trans_b) {
    float* Ar = round_pack_a(A, row0, nrows, K, lda);
    float* Br = round_pack_b(B, K, N, ldb, trans_b);
    if (C32) gemm_rows_f32(Ar, Br, C32, nrows, N, K, N);
    if (C64) gemm_rows_f64(Ar, Br, C64, nrows, N, K, N);
    free(Ar);
    free(Br);
}

/* ------------------------------------------------------------------------- */
/* Batched driver with broadcast: src/OperationKernels.cu:914-1026.           */
/* ------------------------------------------------------------------------- */
static size_t stride0(const size_t s[4]) { return s[1] * s[2] * s[3]; }   /* Dimension.cu:5-10 */
static size_t stride1(const size_t s[4]) { return s[2] * s[3]; }

void nzo_tensorcore_gemm(const float* A, const float* B, float* C, const size_t shapeA[4],
                         const size_t shapeB[4], const size_t shapeC[4]) {
    const size_t M = shapeA[2], N = shapeB[3], K = shapeA[3];           /* :918-920 */
    for (size_t i = 0; i < shapeC[0]; i++) {                             /* :978-986 */
        for (size_t j = 0; j < shapeC[1]; j++) {
            const size_t oc = i * stride0(shapeC) + j * stride1(shapeC);
            const size_t oa = i * (shapeA[0] > 1 ? stride0(shapeA) : 0) + j * (shapeA[1] > 1 ? stride1(shapeA) : 0);
            const size_t ob = i * (shapeB[0] > 1 ? stride0(shapeB) : 0) + j * (shapeB[1] > 1 ? stride1(shapeB) : 0);
            nzo_gemm_f16in_f32acc(A + oa, B + ob, C + oc, M, N, K, K, N, N, 0);
        }
    }
}

/* fp32-exact comparator: src/OperationKernels.cu:65-101 via
 * include/NeuZephyr/TensorOperations.cuh:998-1019 (same offsets, no rounding). */
void nzo_general_matmul(const float* A, const float* B, float* C, const size_t shapeA[4],
                        const size_t shapeB[4], const size_t shapeC[4]) {
    const size_t M = shapeA[2], N = shapeB[3], K = shapeA[3];
    for (size_t i = 0; i < shapeC[0]; i++) {
        for (size_t j = 0; j < shapeC[1]; j++) {
            const float* a = A + i * (shapeA[0] > 1 ? stride0(shapeA) : 0) + j * (shapeA[1] > 1 ? stride1(shapeA) : 0);
            const float* b = B + i * (shapeB[0] > 1 ? stride0(shapeB) : 0) + j * (shapeB[1] > 1 ? stride1(shapeB) : 0);
            float* c = C + i * stride0(shapeC) + j * stride1(shapeC);
            for (size_t r = 0; r < M; r++)
                for (size_t q = 0; q < N; q++) {
                    float sum = 0.0f;
                    /* nvcc contracts `sum += As*Bs` (:92-93) into one FMA per k (its default -fmad=true) */
                    for (size_t k = 0; k < K; k++) sum = fmaf(a[r * K + k], b[k * N + q], sum);
                    c[r * N + q] = sum;
                }
        }
    }
}

/* ------------------------------------------------------------------------- */
/* im2col: src/OperationKernels.cu:1308-1328, index by index.                 */
/* ------------------------------------------------------------------------- */
void nzo_im2col(float* out, const float* in, size_t H_out, size_t W_out, size_t C, size_t K_h,
                size_t K_w, size_t stride, size_t pad, size_t H_in, size_t W_in, size_t batch) {
    const size_t per = H_out * W_out * C * K_h * K_w;
    const size_t total = per * batch;
#pragma omp parallel for schedule(static)
    for (size_t idx = 0; idx < total; idx++) {
        const size_t fixedIdx = idx % per;                                /* :1315 */
        const size_t currentBatch = idx / per;                            /* :1316 */
        const size_t k = fixedIdx / (C * K_h * K_w);                      /* output pixel */
        const size_t m = fixedIdx % (C * K_h * K_w);                      /* column = c*Kh*Kw + r*Kw + s */
        const size_t c = m / (K_h * K_w);
        const long long h = (long long)((k / W_out) * stride) - (long long)pad + (long long)((m % (K_h * K_w)) / K_w);
        const long long w = (long long)((k % W_out) * stride) - (long long)pad + (long long)(m % K_w);
        if (h >= 0 && h < (long long)H_in && w >= 0 && w < (long long)W_in)
            out[idx] = in[currentBatch * (C * H_in * W_in) + c * (H_in * W_in) + (size_t)h * W_in + (size_t)w];
        else
            out[idx] = 0.0f;
    }
}

/* col2im: src/OperationKernels.cu:1364-1376. */
void nzo_col2im(float* out, const float* in, size_t H_out, size_t W_out, size_t C_out, size_t batches) {
    const size_t per = C_out * H_out * W_out;
    const size_t total = per * batches;
#pragma omp parallel for schedule(static)
    for (size_t idx = 0; idx < total; idx++) {
        const size_t batch = idx / per;
        const size_t fixedIdx = idx % per;
        const size_t c = fixedIdx / (H_out * W_out);
        const size_t h = (fixedIdx % (H_out * W_out)) / W_out;
        const size_t w = (fixedIdx % (H_out * W_out)) % W_out;
        out[idx] = in[batch * per + (h * W_out + w) * C_out + c];
    }
}

/* Broadcast add: include/NeuZephyr/TensorOperations.cuh:785-808 (offsets) +
 * src/OperationKernels.cu:12-24 (kernel). H and W must agree. */
void nzo_matrix_add(float* out, const float* a, const float* b, const size_t shapeOut[4],
                    const size_t shapeA[4], const size_t shapeB[4]) {
    const size_t n = shapeA[2] * shapeA[3];
    for (size_t i = 0; i < shapeOut[0]; i++) {
        for (size_t j = 0; j < shapeOut[1]; j++) {
            float* c_m = out + i * stride0(shapeOut) + j * stride1(shapeOut);
            const float* a_m = a + i * (shapeA[0] > 1 ? stride0(shapeA) : 0) + j * (shapeA[1] > 1 ? stride1(shapeA) : 0);
            const float* b_m = b + i * (shapeB[0] > 1 ? stride0(shapeB) : 0) + j * (shapeB[1] > 1 ? stride1(shapeB) : 0);
            for (size_t idx = 0; idx < n; idx++) c_m[idx] = a_m[idx] + b_m[idx];
        }
    }
}

/* ReLU: src/OperationKernels.cu:230-235. NaN > 0 is false -> 0; -0 -> 0. */
void nzo_relu(float* out, const float* in, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; i++) out[i] = in[i] > 0 ? in[i] : 0;
}

/* ------------------------------------------------------------------------- */
/* Backward of the path.                                                      */
/* ------------------------------------------------------------------------- */
/* src/OperationKernels.cu:1028-1144: same M/N/K and offsets as the forward driver, the batch
 * runs over max(A,B) and a C dimension of 1 collects every member (CuttingAndCompress). */
void nzo_gemm_backward(const float* A, const float* B, float* C, const size_t shapeA[4],
                       const size_t shapeB[4], const size_t shapeC[4]) {
    const size_t M = shapeA[2], N = shapeB[3], K = shapeA[3];
    const size_t bn = shapeA[0] > shapeB[0] ? shapeA[0] : shapeB[0];
    const size_t bc = shapeA[1] > shapeB[1] ? shapeA[1] : shapeB[1];
    float* tmp = (float*)malloc((M * N > 0 ? M * N : 1) * sizeof(float));
    for (size_t i = 0; i < bn; i++) {
        for (size_t j = 0; j < bc; j++) {
            const size_t oa = i * (shapeA[0] > 1 ? stride0(shapeA) : 0) + j * (shapeA[1] > 1 ? stride1(shapeA) : 0);
            const size_t ob = i * (shapeB[0] > 1 ? stride0(shapeB) : 0) + j * (shapeB[1] > 1 ? stride1(shapeB) : 0);
            const size_t oc = i * (shapeC[0] > 1 ? stride0(shapeC) : 0) + j * (shapeC[1] > 1 ? stride1(shapeC) : 0);
            nzo_gemm_f16in_f32acc(A + oa, B + ob, tmp, M, N, K, K, N, N, 0);
            for (size_t e = 0; e < M * N; e++) C[oc + e] += tmp[e];      /* :873-883 */
        }
    }
    free(tmp);
}

static void transpose_batched(float* dst, const float* src, const size_t shape[4]) {   /* :125-145 */
    const size_t R = shape[2], Cn = shape[3], nb = shape[0] * shape[1];
    for (size_t b = 0; b < nb; b++)
        for (size_t r = 0; r < R; r++)
            for (size_t c = 0; c < Cn; c++) dst[b * R * Cn + c * R + r] = src[b * R * Cn + r * Cn + c];
}

void nzo_matmul_backward(float* dA, float* dB, const float* A, const float* B, const float* dC,
                         const size_t shapeA[4], const size_t shapeB[4], const size_t shapeC[4]) {
    if (dA) {                                                          /* Nodes.cu:171-175 */
        const size_t nB = shapeB[0] * shapeB[1] * shapeB[2] * shapeB[3];
        float* bt = (float*)malloc((nB ? nB : 1) * sizeof(float));
        const size_t shapeBT[4] = {shapeB[0], shapeB[1], shapeB[3], shapeB[2]};
        transpose_batched(bt, B, shapeB);
        nzo_gemm_backward(dC, bt, dA, shapeC, shapeBT, shapeA);
        free(bt);
    }
    if (dB) {                                                          /* Nodes.cu:177-181 */
        const size_t nA = shapeA[0] * shapeA[1] * shapeA[2] * shapeA[3];
        float* at = (float*)malloc((nA ? nA : 1) * sizeof(float));
        const size_t shapeAT[4] = {shapeA[0], shapeA[1], shapeA[3], shapeA[2]};
        transpose_batched(at, A, shapeA);
        nzo_gemm_backward(at, dC, dB, shapeAT, shapeC, shapeB);
        free(at);
    }
}

void nzo_relu_backward(float* dx, const float* x, const float* dy, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; i++) dx[i] = x[i] > 0 ? dy[i] : 0;
}

void nzo_add_backward(float* din, const float* dout, const size_t shapeIn[4], const size_t shapeOut[4]) {
    const size_t n = shapeOut[2] * shapeOut[3];
    if (shapeIn[0] == shapeOut[0] && shapeIn[1] == shapeOut[1] && shapeIn[2] == shapeOut[2] &&
        shapeIn[3] == shapeOut[3]) {                                   /* Nodes.cu:101-105: memcpy */
        memcpy(din, dout, shapeOut[0] * shapeOut[1] * n * sizeof(float));
        return;
    }
    for (size_t i = 0; i < shapeOut[0]; i++)                           /* Nodes.cu:107-121 */
        for (size_t j = 0; j < shapeOut[1]; j++) {
            const float* src = dout + i * stride0(shapeOut) + j * stride1(shapeOut);
            float* dst = din + i * (shapeIn[0] > 1 ? stride0(shapeIn) : 0) + j * (shapeIn[1] > 1 ? stride1(shapeIn) : 0);
            for (size_t idx = 0; idx < n; idx++) dst[idx] += src[idx];
        }
}

void nzo_im2col_backward(float* dx, const float* dcol, size_t H_out, size_t W_out, size_t C, size_t K_h,
                         size_t K_w, size_t stride, size_t pad, size_t H_in, size_t W_in, size_t batch) {
    const size_t per = H_out * W_out * C * K_h * K_w;
    for (size_t idx = 0; idx < per * batch; idx++) {                   /* :1341-1354, index by index */
        const size_t fixedIdx = idx % per, currentBatch = idx / per;
        const size_t k = fixedIdx / (C * K_h * K_w), m = fixedIdx % (C * K_h * K_w);
        const size_t c = m / (K_h * K_w);
        const long long h = (long long)((k / W_out) * stride) - (long long)pad + (long long)((m % (K_h * K_w)) / K_w);
        const long long w = (long long)((k % W_out) * stride) - (long long)pad + (long long)(m % K_w);
        if (h >= 0 && h < (long long)H_in && w >= 0 && w < (long long)W_in)
            dx[currentBatch * (C * H_in * W_in) + c * (H_in * W_in) + (size_t)h * W_in + (size_t)w] += dcol[idx];
    }
}

void nzo_col2im_backward(float* dcol, const float* dy, size_t H_out, size_t W_out, size_t C_out, size_t batches) {
    const size_t per = C_out * H_out * W_out;
#pragma omp parallel for schedule(static)
    for (size_t idx = 0; idx < per * batches; idx++) {                 /* :1386-1395 */
        const size_t batch = idx / per, fixedIdx = idx % per;
        const size_t c = fixedIdx / (H_out * W_out);
        const size_t h = (fixedIdx % (H_out * W_out)) / W_out, w = (fixedIdx % (H_out * W_out)) % W_out;
        dcol[batch * per + (h * W_out + w) * C_out + c] = dy[idx];
    }
}

/* Data gradient of the Model::Conv2d graph in one statement. The reference computes it
 * as the chain Col2ImgNode::backward (src/Nodes.cu:660-665) -> MatMulNode::backward, dA += dC * B^T
 * with fp16-rounded operands and fp32 accumulation (:169-182) -> Img2ColNode::backward (:632-640,
 * img2colBackwardKernel, src/OperationKernels.cu:1337-1362). Composed:
 *   dx[b][c][h][w] += sum over r, s, o of f16(dy[b][o][ho][wo]) * f16(W[wb][(c,r,s)][o])
 * for the (r, s) with ho * stride = h + pad - r and wo * stride = w + pad - s inside the output. Here o runs
 * innermost in ascending order inside each (r, s), then the taps in ascending (r, s): the grouping of the
 * chain (a dot product over o per column-matrix entry, then one addition per tap). */
void nzo_conv2d_backward_data_strided(float* dx, const float* dy, const float* w_ref, size_t N, size_t C, size_t H,
                                      size_t W, size_t O, size_t K_h, size_t K_w, size_t stride, size_t pad,
                                      size_t w_batch) {
    const size_t H_out = (H + 2 * pad - K_h) / stride + 1, W_out = (W + 2 * pad - K_w) / stride + 1, CKK = C * K_h * K_w;
    float* dyr = (float*)malloc(sizeof(float) * N * O * H_out * W_out);
    float* wr = (float*)malloc(sizeof(float) * w_batch * CKK * O);
    nzo_round_f16_array(dyr, dy, N * O * H_out * W_out);
    nzo_round_f16_array(wr, w_ref, w_batch * CKK * O);
#pragma omp parallel for collapse(2) schedule(static)
    for (size_t b = 0; b < N; b++)
        for (size_t c = 0; c < C; c++) {
            const float* wb = wr + (w_batch > 1 ? b : 0) * CKK * O;
            for (size_t h = 0; h < H; h++)
                for (size_t w = 0; w < W; w++) {
                    float g = dx[((b * C + c) * H + h) * W + w];
                    for (size_t r = 0; r < K_h; r++)
                        for (size_t s = 0; s < K_w; s++) {
                            const long long hs = (long long)(h + pad) - (long long)r, ws = (long long)(w + pad) - (long long)s;
                            if (hs < 0 || ws < 0 || hs % (long long)stride || ws % (long long)stride) continue;
                            const long long ho = hs / (long long)stride, wo = ws / (long long)stride;
                            if (ho >= (long long)H_out || wo >= (long long)W_out) continue;
                            const float* wrow = wb + ((c * K_h + r) * K_w + s) * O;
                            float dot = 0.0f;
                            for (size_t o = 0; o < O; o++)
                                dot += dyr[((b * O + o) * H_out + (size_t)ho) * W_out + (size_t)wo] * wrow[o];
                            g += dot;
                        }
                    dx[((b * C + c) * H + h) * W + w] = g;
                }
        }
    free(dyr);
    free(wr);
}

void nzo_conv2d_backward_data(float* dx, const float* dy, const float* w_ref, size_t N, size_t C, size_t H,
                              size_t W, size_t O, size_t K_h, size_t K_w, size_t pad, size_t w_batch) {
    nzo_conv2d_backward_data_strided(dx, dy, w_ref, N, C, H, W, O, K_h, K_w, 1, pad, w_batch);
}

/* Weight gradient of the Model::Conv2d graph in one statement: MatMulNode::backward's
 * dB += A^T * dC (src/Nodes.cu:169-182) with A the column matrix of Img2ColNode::forward (:605-630,
 * img2colKernel src/OperationKernels.cu:1308-1328: h = ho*stride - pad + r, w = wo*stride - pad + s) and dC the
 * pixel-major gradient of Col2ImgNode::backward (:660-665); fp16-rounded operands, fp32 accumulation over the
 * pixels in ascending order (and over the images, for shared weights). */
void nzo_conv2d_backward_weights_strided(float* dw, const float* x, const float* dy, size_t N, size_t C, size_t H,
                                         size_t W, size_t O, size_t K_h, size_t K_w, size_t stride, size_t pad,
                                         size_t w_batch) {
    const size_t H_out = (H + 2 * pad - K_h) / stride + 1, W_out = (W + 2 * pad - K_w) / stride + 1, CKK = C * K_h * K_w;
    float* xr = (float*)malloc(sizeof(float) * N * C * H * W);
    float* dyr = (float*)malloc(sizeof(float) * N * O * H_out * W_out);
    nzo_round_f16_array(xr, x, N * C * H * W);
    nzo_round_f16_array(dyr, dy, N * O * H_out * W_out);
#pragma omp parallel for collapse(2) schedule(static)
    for (size_t q = 0; q < CKK; q++)
        for (size_t o = 0; o < O; o++) {
            const size_t c = q / (K_h * K_w), r = (q % (K_h * K_w)) / K_w, s = q % K_w;
            for (size_t wb = 0; wb < w_batch; wb++) {
                float acc = 0.0f;
                for (size_t b = (w_batch > 1 ? wb : 0); b < (w_batch > 1 ? wb + 1 : N); b++)
                    for (size_t ho = 0; ho < H_out; ho++)
                        for (size_t wo = 0; wo < W_out; wo++) {
                            const long long h = (long long)(ho * stride + r) - (long long)pad,
                                            w = (long long)(wo * stride + s) - (long long)pad;
                            if (h < 0 || h >= (long long)H || w < 0 || w >= (long long)W) continue;
                            acc += xr[((b * C + c) * H + (size_t)h) * W + (size_t)w] * dyr[((b * O + o) * H_out + ho) * W_out + wo];
                        }
                dw[(wb * CKK + q) * O + o] += acc;
            }
        }
    free(xr);
    free(dyr);
}

void nzo_conv2d_backward_weights(float* dw, const float* x, const float* dy, size_t N, size_t C, size_t H, size_t W,
                                 size_t O, size_t K_h, size_t K_w, size_t pad, size_t w_batch) {
    nzo_conv2d_backward_weights_strided(dw, x, dy, N, C, H, W, O, K_h, K_w, 1, pad, w_batch);
}

/* ------------------------------------------------------------------------- */
/* Softmax and its Jacobian: test/Test.cpp:1823-1832 and :1782-1795.          */
/* ------------------------------------------------------------------------- */
void nzo_softmax(float* out, const float* in, size_t len, size_t batch) {
    for (size_t b = 0; b < batch; b++) {
        float sum = 0.0f;
        for (size_t k = 0; k < len; k++) sum += expf(in[b * len + k]);
        for (size_t k = 0; k < len; k++) out[b * len + k] = expf(in[b * len + k]) / sum;
    }
}

void nzo_softmax_jacobian(float* out, const float* in, size_t n, size_t batch) {
    for (size_t b = 0; b < batch; b++)
        for (size_t x = 0; x < n; x++)
            for (size_t y = 0; y < n; y++)
                out[b * n * n + x * n + y] = x == y ? in[b * n + x] * (1 - in[b * n + x]) : -in[b * n + x] * in[b * n + y];
}

/* ------------------------------------------------------------------------- */
/* Optimizer steps: src/OperationKernels.cu:634-640 and :753-766.             */
/* ------------------------------------------------------------------------- */
void nzo_sgd_step(float* data, const float* grad, float lr, size_t n) {
    for (size_t i = 0; i < n; i++) data[i] -= lr * grad[i];
}

void nzo_adam_step(float* data, float* m, float* v, const float* grad, float lr, float beta1, float beta2,
                   float eps, int t, size_t n) {
    const float corr1 = 1.0f - powf(beta1, (float)t), corr2 = 1.0f - powf(beta2, (float)t);
    for (size_t i = 0; i < n; i++) {
        const float m_temp = m[i] * beta1 + grad[i] * (1 - beta1);
        const float v_temp = v[i] * beta2 + grad[i] * grad[i] * (1 - beta2);
        const float m_modified = m_temp / corr1;
        const float v_modified = v_temp / corr2;
        data[i] -= lr * m_modified / (sqrtf(v_modified) + eps);
        m[i] = m_temp;
        v[i] = v_temp;
    }
}

/* ------------------------------------------------------------------------- */
/* Model::Conv2d graph (src/Model.cu:244-263): Img2Col -> MatMul -> Bias(Add)  */
/* -> Col2Img, then an optional ReLU node; intermediates materialised.         */
/* ------------------------------------------------------------------------- */
void nzo_conv2d_graph(float* y, const float* x, const float* w_ref, const float* bias_ref, size_t N,
                      size_t C, size_t H, size_t W, size_t O, size_t K_h, size_t K_w, size_t stride,
                      size_t pad, size_t w_batch, int relu) {
    const size_t H_out = (H + 2 * pad - K_h) / stride + 1;               /* Nodes.cu:605-617 */
    const size_t W_out = (W + 2 * pad - K_w) / stride + 1;
    const size_t HW = H_out * W_out, CKK = C * K_h * K_w;
    float* col = (float*)malloc(sizeof(float) * N * HW * CKK);
    float* res = (float*)malloc(sizeof(float) * N * HW * O);
    nzo_im2col(col, x, H_out, W_out, C, K_h, K_w, stride, pad, H, W, N);
    const size_t sA[4] = {N, 1, HW, CKK}, sB[4] = {w_batch, 1, CKK, O}, sC[4] = {N, 1, HW, O};
    nzo_tensorcore_gemm(col, w_ref, res, sA, sB, sC);
    if (bias_ref) {
        const size_t sBias[4] = {1, 1, HW, O};                           /* Model.cu:68-75 */
        float* tmp = (float*)malloc(sizeof(float) * N * HW * O);
        nzo_matrix_add(tmp, res, bias_ref, sC, sC, sBias);
        free(res);
        res = tmp;
    }
    nzo_col2im(y, res, H_out, W_out, O, N);
    if (relu) nzo_relu(y, y, N * O * HW);
    free(col);
    free(res);
}

/* Independent direct convolution, fp64 accumulation, OIHW weights. */
void nzo_conv2d_direct_f64(double* y, const float* x, const float* w_oihw, const float* bias_o,
                           size_t N, size_t C, size_t H, size_t W, size_t O, size_t K_h, size_t K_w,
                           size_t stride, size_t pad, int relu) {
    const size_t H_out = (H + 2 * pad - K_h) / stride + 1;
    const size_t W_out = (W + 2 * pad - K_w) / stride + 1;
#pragma omp parallel for collapse(2) schedule(static)
    for (size_t b = 0; b < N; b++)
        for (size_t o = 0; o < O; o++)
            for (size_t ho = 0; ho < H_out; ho++)
                for (size_t wo = 0; wo < W_out; wo++) {
                    double acc = 0.0;
                    for (size_t c = 0; c < C; c++)
                        for (size_t r = 0; r < K_h; r++)
                            for (size_t s = 0; s < K_w; s++) {
                                const long long h = (long long)(ho * stride + r) - (long long)pad;
                                const long long w = (long long)(wo * stride + s) - (long long)pad;
                                if (h < 0 || h >= (long long)H || w < 0 || w >= (long long)W) continue;
                                acc += (double)nzo_round_f16(x[((b * C + c) * H + (size_t)h) * W + (size_t)w]) *
                                       (double)nzo_round_f16(w_oihw[((o * C + c) * K_h + r) * K_w + s]);
                            }
                    if (bias_o) acc += (double)bias_o[o];
                    if (relu) acc = acc > 0 ? acc : 0;
                    y[((b * O + o) * H_out + ho) * W_out + wo] = acc;
                }
}

/* ------------------------------------------------------------------------- */
/* Model::Linear graph (src/Model.cu:87-103): Reshape -> MatMul(W[1,1,OUT,IN], */
/* x[N,1,IN,1]) -> Bias([1,1,OUT,1]) (-> ReLU).  Each sample is a GEMV with    */
/* the same k-ascending fp32 sum.                                              */
/* ------------------------------------------------------------------------- */
void nzo_linear_graph(float* y, const float* x, const float* w_out_in, const float* bias, size_t batch,
                      size_t in_features, size_t out_features, int relu) {
    /* y^T[OUT, batch] = W[OUT,IN] * x^T[IN,batch]: identical per-element k order. */
    float* Wr = (float*)malloc(sizeof(float) * out_features * in_features);
    float* Xr = (float*)malloc(sizeof(float) * batch * in_features);
    nzo_round_f16_array(Wr, w_out_in, out_features * in_features);
    nzo_round_f16_array(Xr, x, batch * in_features);
#pragma omp parallel for schedule(static)
    for (size_t n = 0; n < batch; n++) {
        for (size_t o = 0; o < out_features; o++) {
            float acc = 0.0f;
            const float* wr = Wr + o * in_features;
            const float* xr = Xr + n * in_features;
            for (size_t k = 0; k < in_features; k++) acc += wr[k] * xr[k];
            if (bias) acc = acc + bias[o];
            if (relu) acc = acc > 0 ? acc : 0;
            y[n * out_features + o] = acc;
        }
    }
    free(Wr);
    free(Xr);
}

/* ------------------------------------------------------------------------- */
void nzo_errors_f32_vs_f64(const float* got, const double* truth, size_t n, double floor_abs,
                           double* max_rel, double* frob_rel) {
    double mr = 0.0, num = 0.0, den = 0.0;
#pragma omp parallel for reduction(max : mr) reduction(+ : num, den) schedule(static)
    for (size_t i = 0; i < n; i++) {
        const double d = fabs((double)got[i] - truth[i]);
        const double t = fabs(truth[i]);
        const double r = d / (t > floor_abs ? t : floor_abs);
        if (r > mr || r != r) mr = (r != r) ? INFINITY : r;
        num += d * d;
        den += truth[i] * truth[i];
    }
    if (max_rel) *max_rel = mr;
    if (frob_rel) *frob_rel = den > 0 ? sqrt(num / den) : sqrt(num);
}

/* ------------------------------------------------------------------------- */
/* Seeded generators.                                                         */
/* ------------------------------------------------------------------------- */
static inline uint64_t splitmix64(uint64_t* s) {
    uint64_t z = (*s += 0x9e3779b97f4a7c15ull);
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}
static inline uint64_t rotl64(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }
static inline uint64_t xoshiro_next(uint64_t s[4]) {
    const uint64_t result = rotl64(s[1] * 5, 7) * 9;
    const uint64_t t = s[1] << 17;
    s[2] ^= s[0];
    s[3] ^= s[1];
    s[1] ^= s[2];
    s[0] ^= s[3];
    s[2] ^= t;
    s[3] = rotl64(s[3], 45);
    return result;
}
static inline double u01(uint64_t s[4]) { return (double)(xoshiro_next(s) >> 11) * (1.0 / 9007199254740992.0); }

#define NZO_FILL_BLOCK 4096

void nzo_fill(float* dst, size_t n, uint64_t seed, int kind, double lo, double hi) {
    const size_t nblocks = (n + NZO_FILL_BLOCK - 1) / NZO_FILL_BLOCK;
#pragma omp parallel for schedule(static)
    for (size_t blk = 0; blk < nblocks; blk++) {
        uint64_t sm = seed * 0xd1342543de82ef95ull + blk * 0x2545f4914f6cdd1dull + 0x1234567ull;
        uint64_t s[4];
        for (int i = 0; i < 4; i++) s[i] = splitmix64(&sm);
        const size_t i0 = blk * NZO_FILL_BLOCK;
        const size_t i1 = i0 + NZO_FILL_BLOCK < n ? i0 + NZO_FILL_BLOCK : n;
        if (kind == 0) {
            for (size_t i = i0; i < i1; i++) dst[i] = (float)(lo + (hi - lo) * u01(s));
        } else {
            for (size_t i = i0; i < i1; i += 2) {
                double u1 = u01(s), u2 = u01(s);
                if (u1 < 1e-300) u1 = 1e-300;
                const double r = sqrt(-2.0 * log(u1));
                const double th = 6.283185307179586476925286766559 * u2;
                dst[i] = (float)(lo + hi * r * cos(th));
                if (i + 1 < i1) dst[i + 1] = (float)(lo + hi * r * sin(th));
            }
        }
    }
}

void nzo_avgpool2d(float* out, const float* in, size_t pool, size_t stride, size_t pad, size_t batches,
                   size_t channels, size_t H_in, size_t W_in, size_t H_out, size_t W_out) {
    for (size_t pl = 0; pl < batches * channels; pl++)
        for (size_t h = 0; h < H_out; h++)
            for (size_t w = 0; w < W_out; w++) {
                const long long h0 = (long long)(h * stride) - (long long)pad, w0 = (long long)(w * stride) - (long long)pad;
                float sum = 0.0f;
                size_t count = 0;
                for (size_t i = 0; i < pool; i++)
                    for (size_t j = 0; j < pool; j++) {
                        const long long hi = h0 + (long long)i, wi = w0 + (long long)j;
                        if (hi >= 0 && hi < (long long)H_in && wi >= 0 && wi < (long long)W_in) {
                            sum += in[pl * H_in * W_in + (size_t)hi * W_in + (size_t)wi];
                            count++;
                        }
                    }
                out[pl * H_out * W_out + h * W_out + w] = count > 0 ? sum / (float)count : 0.0f;
            }
}

void nzo_avgpool2d_backward(float* din, const float* dout, size_t pool, size_t stride, size_t pad, size_t batches,
                            size_t channels, size_t H_in, size_t W_in, size_t H_out, size_t W_out) {
    for (size_t pl = 0; pl < batches * channels; pl++)
        for (size_t h = 0; h < H_out; h++)
            for (size_t w = 0; w < W_out; w++) {
                const long long h0 = (long long)(h * stride) - (long long)pad, w0 = (long long)(w * stride) - (long long)pad;
                size_t count = 0;
                for (size_t i = 0; i < pool; i++)
                    for (size_t j = 0; j < pool; j++) {
                        const long long hi = h0 + (long long)i, wi = w0 + (long long)j;
                        if (hi >= 0 && hi < (long long)H_in && wi >= 0 && wi < (long long)W_in) count++;
                    }
                const float g = dout[pl * H_out * W_out + h * W_out + w];
                const float div = pad == 0 ? (float)(pool * pool) : (float)count;
                for (size_t i = 0; i < pool; i++)
                    for (size_t j = 0; j < pool; j++) {
                        const long long hi = h0 + (long long)i, wi = w0 + (long long)j;
                        if (hi >= 0 && hi < (long long)H_in && wi >= 0 && wi < (long long)W_in)
                            din[pl * H_in * W_in + (size_t)hi * W_in + (size_t)wi] += g / div;
                    }
            }
}

float nzo_bce_loss(const float* predict, const float* real, size_t n) {
    float loss = 0.0f;
    for (size_t i = 0; i < n; i++) loss += -real[i] * logf(predict[i]) - (1 - real[i]) * logf(1 - predict[i]);
    return n ? loss / (float)n : 0.0f;
}

void nzo_bce_backward(float* grad, const float* predict, const float* real, size_t n) {
    for (size_t i = 0; i < n; i++) grad[i] = ((predict[i] - real[i]) / (predict[i] * (1 - predict[i]))) / (float)n;
}

float nzo_mse_loss(const float* predict, const float* real, size_t n) {
    float loss = 0.0f;
    for (size_t i = 0; i < n; i++) loss += (predict[i] - real[i]) * (predict[i] - real[i]);
    return n ? loss / (float)n : 0.0f;
}

void nzo_mse_backward(float* grad, const float* predict, const float* real, size_t n) {
    for (size_t i = 0; i < n; i++) grad[i] = 2 * (predict[i] - real[i]) / (float)n;
}

void nzo_expand(float* out, const float* in, size_t n, size_t batches) {
    for (size_t i = 0; i < n * batches; i++) out[i] = in[i % n];
}

void nzo_compress(float* out, const float* in, size_t n, size_t batches) {
    for (size_t i = 0; i < n * batches; i++) out[i % n] += in[i];
}

int nzo_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void nzo_set_num_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}
