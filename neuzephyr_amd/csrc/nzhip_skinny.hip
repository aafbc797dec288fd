// Bandwidth-bound GEMM kernels for products with very few rows or columns (min(M, N) <= 8; which of
// those shapes come here is decided in gemm_skinny_applicable):
// GEMV-shaped work such as one sample through Model::Linear or the M = 1 case of
// TensorCoreGEMMParallel (src/OperationKernels.cu:914-1026), where an MFMA tile would be >= 75 %
// padding and the reference pads 1 row up to 16 (:921-923). The big operand is streamed from
// HBM exactly once with 16-byte loads; both operands are rounded to fp16 (RNE) on the fly and
// products are accumulated in fp32, as the tensor-core path does.
//
// Formulation: out(s, l) = sum_k S(s, k) * L(k, l), s < SR <= 8 ("skinny" side), l the long side.
//   KL kernel: L is stored with l contiguous  (L(k,l) at L[k*ld + l]); lanes own 4 adjacent l,
//              waves and grid.y split k; partial sums meet in LDS, then (if k is split over
//              blocks) in a workspace that a small second kernel reduces deterministically.
//   LK kernel: L is stored with k contiguous  (L(k,l) at L[l*ld + k]); a wave owns 4 rows l,
//              lanes stride k, and the 64 partial sums are folded with cross-lane shuffles.
#include <hip/hip_runtime.h>

#include <cstdlib>

#include "nzhip_internal.h"

namespace nzhip {

typedef float floatx4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float rnd16(float x) { return (float)(_Float16)x; }

struct SkinnyArgs {
    const float* S;
    const float* L;
    float* out;
    const float* bias;
    int SR, LN, K;                  // skinny rows, long extent, reduction extent
    long s_ss, s_sk;                // S(s,k) at S[s*s_ss + k*s_sk]
    long ldl;                       // leading dimension of L
    long o_ss, o_sl;                // out(s,l) at out[s*o_ss + l*o_sl]
    long b_ss, b_sl;                // bias strides
    int batch_c;
    long S_sn, S_sc, L_sn, L_sc, o_sn, o_sc, b_sn, b_sc;
    int relu;
    int ksplit, kslice;             // KL: blocks along k and k per block
    float* partial;                 // KL with ksplit > 1: [batch][ksplit][SR][LN]
    int vec;
};

// ---- KL: stream rows of L -------------------------------------------------------------------
template <int SR>
__global__ __launch_bounds__(256) void skinny_kl_kernel(const SkinnyArgs p) {
    __shared__ float red[4][SR][256];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int bz = blockIdx.z, bi = bz / p.batch_c, bj = bz % p.batch_c;
    const float* __restrict__ S = p.S + bi * p.S_sn + bj * p.S_sc;
    const float* __restrict__ L = p.L + bi * p.L_sn + bj * p.L_sc;
    const int l0 = (blockIdx.x * 64 + lane) * 4;
    const int kb = blockIdx.y * p.kslice;
    const int ke = (kb + p.kslice < p.K) ? kb + p.kslice : p.K;

    float acc[SR][4];
#pragma unroll
    for (int s = 0; s < SR; s++)
#pragma unroll
        for (int e = 0; e < 4; e++) acc[s][e] = 0.f;

    const bool in_l = l0 < p.LN;
    const bool full = p.vec && (l0 + 4 <= p.LN);
    // waves interleave k so that the four of them read four adjacent rows at a time
    for (int k = kb + wave; k < ke; k += 4) {
        floatx4 v = {0.f, 0.f, 0.f, 0.f};
        const float* row = L + (long)k * p.ldl;
        if (full) {
            v = *reinterpret_cast<const floatx4*>(row + l0);
        } else if (in_l) {
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (l0 + e < p.LN) v[e] = row[l0 + e];
        }
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = rnd16(v[e]);
#pragma unroll
        for (int s = 0; s < SR; s++) {
            const float a = (s < p.SR) ? rnd16(S[s * p.s_ss + k * p.s_sk]) : 0.f;   // wave-uniform address
#pragma unroll
            for (int e = 0; e < 4; e++) acc[s][e] = __builtin_fmaf(a, v[e], acc[s][e]);
        }
    }
    // fold the four waves
#pragma unroll
    for (int s = 0; s < SR; s++)
#pragma unroll
        for (int e = 0; e < 4; e++) red[wave][s][lane * 4 + e] = acc[s][e];
    __syncthreads();
    for (int idx = threadIdx.x; idx < SR * 256; idx += 256) {
        const int s = idx / 256, c = idx % 256;
        const int l = blockIdx.x * 256 + c;
        if (s >= p.SR || l >= p.LN) continue;
        const float v = (red[0][s][c] + red[1][s][c]) + (red[2][s][c] + red[3][s][c]);
        if (p.ksplit > 1) {
            p.partial[(((long)bz * p.ksplit + blockIdx.y) * p.SR + s) * p.LN + l] = v;
        } else {
            float x = v;
            if (p.bias) x += p.bias[bi * p.b_sn + bj * p.b_sc + s * p.b_ss + l * p.b_sl];
            if (p.relu) x = x > 0.f ? x : 0.f;
            p.out[bi * p.o_sn + bj * p.o_sc + s * p.o_ss + l * p.o_sl] = x;
        }
    }
}

__global__ __launch_bounds__(256) void skinny_reduce_kernel(const SkinnyArgs p) {
    // 64 outputs per block; the 4 waves take interleaved partials (fixed order => deterministic),
    // loads are independent so they pipeline, and LDS folds the 4 wave sums.
    __shared__ float red[4][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long t = (long)blockIdx.x * 64 + lane;
    const long total = (long)p.SR * p.LN;
    const int bz = blockIdx.z, bi = bz / p.batch_c, bj = bz % p.batch_c;
    float x = 0.f;
    if (t < total) {
        const float* src = p.partial + (long)bz * p.ksplit * total + t;
#pragma unroll 8
        for (int q = wave; q < p.ksplit; q += 4) x += src[(long)q * total];
    }
    red[wave][lane] = x;
    __syncthreads();
    if (wave == 0 && t < total) {
        const int s = (int)(t / p.LN), l = (int)(t % p.LN);
        x = (red[0][lane] + red[1][lane]) + (red[2][lane] + red[3][lane]);
        if (p.bias) x += p.bias[bi * p.b_sn + bj * p.b_sc + s * p.b_ss + l * p.b_sl];
        if (p.relu) x = x > 0.f ? x : 0.f;
        p.out[bi * p.o_sn + bj * p.o_sc + s * p.o_ss + l * p.o_sl] = x;
    }
}

// ---- KL, whole contraction in one workgroup -------------------------------------------------------
// For one long, wide L (a GEMV against a 4096 x 4096 matrix): a workgroup owns 16 adjacent columns l and the
// WHOLE contraction, so no partial sums leave the chip and no second kernel runs. Eight waves; a thread owns
// four columns (lane & 3) of the rows k = (tid >> 2) + 128 j, so a wave load is sixteen 64-byte row pieces; the
// neighbour workgroup that uses the other half of those 128-byte lines runs on the same XCD (workgroups are
// dealt to the XCDs round-robin, so workgroup i takes column group (i % 8) * (G / 8) + i / 8) and finds them in
// its L2. A thread keeps two sets of U loads in flight (8 waves x 2 U KiB per CU). The 128 row lanes are folded
// through LDS in a fixed order.
constexpr int KLC_COLS = 16, KLC_ROWS = 128, KLC_THREADS = 512, KLC_U = 8;

template <int SR>
__global__ __launch_bounds__(KLC_THREADS) void skinny_kl_cols_kernel(const SkinnyArgs p) {
    __shared__ float red[SR][KLC_ROWS][KLC_COLS + 1];
    const int tid = threadIdx.x, q = tid & 3, rl = tid >> 2;
    const int G = gridDim.x;
    const int g = (G % 8 == 0) ? (blockIdx.x % 8) * (G / 8) + blockIdx.x / 8 : blockIdx.x;
    const int l0 = g * KLC_COLS + q * 4;
    const float* __restrict__ S = p.S;
    const float* __restrict__ Lp = p.L + l0;

    float acc[SR][4];
#pragma unroll
    for (int s = 0; s < SR; s++)
#pragma unroll
        for (int e = 0; e < 4; e++) acc[s][e] = 0.f;

    // two register sets: the loads of chunk c + 1 are issued before chunk c is added up
    floatx4 v[2][KLC_U];
    float a[2][SR][KLC_U];
    auto request = [&](int kb, int set) {
#pragma unroll
        for (int u = 0; u < KLC_U; u++) {
            const int k = kb + KLC_ROWS * u;
            const int kc = k < p.K ? k : rl;                                   // clamped: a row this thread owns anyway
            v[set][u] = *reinterpret_cast<const floatx4*>(Lp + (long)kc * p.ldl);
#pragma unroll
            for (int s = 0; s < SR; s++) a[set][s][u] = S[s * p.s_ss + kc * p.s_sk];
        }
    };
    auto add_up = [&](int kb, int set) {
#pragma unroll
        for (int u = 0; u < KLC_U; u++) {
            const bool live = kb + KLC_ROWS * u < p.K;
#pragma unroll
            for (int s = 0; s < SR; s++) {
                const float as = live ? rnd16(a[set][s][u]) : 0.f;
#pragma unroll
                for (int e = 0; e < 4; e++) acc[s][e] = __builtin_fmaf(as, rnd16(v[set][u][e]), acc[s][e]);
            }
        }
    };
    constexpr int STEP = KLC_ROWS * KLC_U;
    request(rl, 0);
    for (int kb = rl; kb < p.K; kb += 2 * STEP) {
        request(kb + STEP, 1);                                                 // past the end: clamped loads, nothing added
        add_up(kb, 0);
        request(kb + 2 * STEP, 0);
        add_up(kb + STEP, 1);
    }
#pragma unroll
    for (int s = 0; s < SR; s++)
#pragma unroll
        for (int e = 0; e < 4; e++) red[s][rl][q * 4 + e] = acc[s][e];
    __syncthreads();
    // output (s, c): eight lanes add sixteen row lanes each, ascending, then fold 8 -> 1 in a fixed tree
    if (tid < SR * KLC_COLS * 8) {
        const int part = tid & 7, oc = tid >> 3, s = oc / KLC_COLS, c = oc % KLC_COLS;
        float x = 0.f;
#pragma unroll
        for (int r = 0; r < KLC_ROWS / 8; r++) x += red[s][part * (KLC_ROWS / 8) + r][c];
        x += __shfl_xor(x, 1);
        x += __shfl_xor(x, 2);
        x += __shfl_xor(x, 4);
        if (part == 0) {
            const int l = g * KLC_COLS + c;
            if (p.bias) x += p.bias[s * p.b_ss + l * p.b_sl];
            if (p.relu) x = x > 0.f ? x : 0.f;
            p.out[s * p.o_ss + l * p.o_sl] = x;
        }
    }
}

// ---- LK: rows of L are dot products ------------------------------------------------------------
template <int SR>
__global__ __launch_bounds__(256) void skinny_lk_kernel(const SkinnyArgs p) {
    constexpr int LR = 4;                                          // rows of L per wave
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int bz = blockIdx.z, bi = bz / p.batch_c, bj = bz % p.batch_c;
    const float* __restrict__ S = p.S + bi * p.S_sn + bj * p.S_sc;
    const float* __restrict__ L = p.L + bi * p.L_sn + bj * p.L_sc;
    const int l0 = (blockIdx.x * 4 + wave) * LR;
    if (l0 >= p.LN) return;

    float acc[SR][LR];
#pragma unroll
    for (int s = 0; s < SR; s++)
#pragma unroll
        for (int r = 0; r < LR; r++) acc[s][r] = 0.f;

    const bool s_contig = p.s_sk == 1;
    int k0 = lane * 4;
    // Whole rows with 16-byte loads: U k steps at a time, their U x (SR + LR) loads issued before any is used -- a
    // wave has only 64 KiB to stream, and one step per round trip to memory would leave it waiting for latency.
    if (p.vec && s_contig && (p.SR == 1 || (p.s_ss & 3) == 0) && l0 + LR <= p.LN) {
        constexpr int U = 4;
        for (; k0 + 256 * (U - 1) + 4 <= p.K; k0 += 256 * U) {
            floatx4 sv[U][SR], lv[U][LR];
#pragma unroll
            for (int u = 0; u < U; u++) {
#pragma unroll
                for (int s = 0; s < SR; s++) {
                    const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
                    sv[u][s] = s < p.SR ? *reinterpret_cast<const floatx4*>(S + s * p.s_ss + k0 + 256 * u) : zero;
                }
#pragma unroll
                for (int r = 0; r < LR; r++) lv[u][r] = *reinterpret_cast<const floatx4*>(L + (long)(l0 + r) * p.ldl + k0 + 256 * u);
            }
#pragma unroll
            for (int u = 0; u < U; u++)
#pragma unroll
                for (int r = 0; r < LR; r++)
#pragma unroll
                    for (int s = 0; s < SR; s++)
#pragma unroll
                        for (int e = 0; e < 4; e++) acc[s][r] = __builtin_fmaf(rnd16(sv[u][s][e]), rnd16(lv[u][r][e]), acc[s][r]);
        }
    }
    for (; k0 < p.K; k0 += 256) {
        const bool fullk = p.vec && (k0 + 4 <= p.K);
        floatx4 sv[SR];
#pragma unroll
        for (int s = 0; s < SR; s++) {
            floatx4 v = {0.f, 0.f, 0.f, 0.f};
            if (s < p.SR) {
                const float* q = S + s * p.s_ss + (long)k0 * p.s_sk;
                if (fullk && s_contig && ((p.s_ss & 3) == 0)) {
                    v = *reinterpret_cast<const floatx4*>(q);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (k0 + e < p.K) v[e] = q[e * p.s_sk];
                }
            }
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = rnd16(v[e]);
            sv[s] = v;
        }
#pragma unroll
        for (int r = 0; r < LR; r++) {
            floatx4 v = {0.f, 0.f, 0.f, 0.f};
            if (l0 + r < p.LN) {
                const float* q = L + (long)(l0 + r) * p.ldl + k0;
                if (fullk) {
                    v = *reinterpret_cast<const floatx4*>(q);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (k0 + e < p.K) v[e] = q[e];
                }
            }
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = rnd16(v[e]);
#pragma unroll
            for (int s = 0; s < SR; s++)
#pragma unroll
                for (int e = 0; e < 4; e++) acc[s][r] = __builtin_fmaf(sv[s][e], v[e], acc[s][r]);
        }
    }
#pragma unroll
    for (int s = 0; s < SR; s++)
#pragma unroll
        for (int r = 0; r < LR; r++) {
            float v = acc[s][r];
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
            acc[s][r] = v;
        }
    if (lane == 0) {
#pragma unroll
        for (int s = 0; s < SR; s++)
#pragma unroll
            for (int r = 0; r < LR; r++) {
                const int l = l0 + r;
                if (s >= p.SR || l >= p.LN) continue;
                float x = acc[s][r];
                if (p.bias) x += p.bias[bi * p.b_sn + bj * p.b_sc + s * p.b_ss + l * p.b_sl];
                if (p.relu) x = x > 0.f ? x : 0.f;
                p.out[bi * p.o_sn + bj * p.o_sc + s * p.o_ss + l * p.o_sl] = x;
            }
    }
}

// ---- host side -------------------------------------------------------------------------------
bool gemm_skinny_applicable(const nzhip_gemm_desc& d) {
    const int64_t small = d.M < d.N ? d.M : d.N, big = d.M < d.N ? d.N : d.M;
    // A single product with 3 or more skinny rows is faster through the MFMA kernel with the
    // contraction split over workgroups (4096^2: 20 us for any M <= 8, against 22..35 us here);
    // with N = 3 that kernel would fall back to scalar loads, so 3 columns stay here. Batched
    // and short (K < 512) products have no split contraction and keep the streaming kernel up to 8.
    int64_t lim = (d.batch_n * d.batch_c > 1 || d.K < 512) ? 8 : (d.N < d.M ? 3 : 2);
    static const char* lim_env = getenv("NZHIP_SKINNY_MAX");            // benchmarking only
    if (lim_env) lim = atoi(lim_env);
    return small >= 1 && small <= lim && big >= 1 && d.batch_n * d.batch_c <= 65535;
}

int gemm_skinny_dispatch(const nzhip_gemm_desc& d, hipStream_t stream) {
    const bool a_trans = d.a_layout == NZHIP_LAYOUT_TRANS, b_trans = d.b_layout == NZHIP_LAYOUT_TRANS;
    SkinnyArgs p = {};
    bool l_is_kl;                    // long operand stored with l contiguous
    if (d.M <= d.N) {
        // skinny side = rows of A, long side = columns of B
        p.S = d.A;
        p.L = d.B;
        p.SR = (int)d.M;
        p.LN = (int)d.N;
        p.s_ss = a_trans ? 1 : d.lda;
        p.s_sk = a_trans ? d.lda : 1;
        p.ldl = d.ldb;
        l_is_kl = !b_trans;
        p.o_ss = d.ldc;
        p.o_sl = 1;
        p.b_ss = d.bias_stride_row;
        p.b_sl = d.bias_stride_col;
        p.S_sn = d.a_stride_n; p.S_sc = d.a_stride_c;
        p.L_sn = d.b_stride_n; p.L_sc = d.b_stride_c;
    } else {
        // skinny side = columns of B, long side = rows of A:  out(s=n, l=m) = sum_k B(k,n) A(m,k)
        p.S = d.B;
        p.L = d.A;
        p.SR = (int)d.N;
        p.LN = (int)d.M;
        p.s_ss = b_trans ? d.ldb : 1;
        p.s_sk = b_trans ? 1 : d.ldb;
        p.ldl = d.lda;
        l_is_kl = a_trans;
        p.o_ss = 1;
        p.o_sl = d.ldc;
        p.b_ss = d.bias_stride_col;
        p.b_sl = d.bias_stride_row;
        p.S_sn = d.b_stride_n; p.S_sc = d.b_stride_c;
        p.L_sn = d.a_stride_n; p.L_sc = d.a_stride_c;
    }
    p.out = d.C;
    p.bias = d.bias;
    p.K = (int)d.K;
    p.batch_c = (int)d.batch_c;
    p.o_sn = d.c_stride_n; p.o_sc = d.c_stride_c;
    p.b_sn = d.bias_stride_n; p.b_sc = d.bias_stride_c;
    p.relu = d.activation == NZHIP_ACT_RELU;
    p.vec = ((p.ldl & 3) == 0) && ((reinterpret_cast<uintptr_t>(p.L) & 15) == 0) && ((p.L_sn & 3) == 0) &&
            ((p.L_sc & 3) == 0) && ((reinterpret_cast<uintptr_t>(p.S) & 15) == 0) && ((p.S_sn & 3) == 0) &&
            ((p.S_sc & 3) == 0);
    const unsigned batch = (unsigned)(d.batch_n * d.batch_c);
    const int sr_t = p.SR <= 1 ? 1 : (p.SR <= 2 ? 2 : (p.SR <= 4 ? 4 : 8));
    int rc = NZHIP_OK;
    float* partial = nullptr;
    static const char* klc_env = getenv("NZHIP_SKINNY_COLS");           // benchmarking only: 0 keeps the split-contraction kernels
    const bool klc_on = !klc_env || atoi(klc_env) != 0;
    if (l_is_kl && klc_on && batch == 1 && p.SR <= 2 && p.vec && p.LN % KLC_COLS == 0 && p.LN >= 128 * KLC_COLS && p.K >= 1024) {
        // enough column groups to occupy the chip, a contraction long enough to stream: one kernel, no partial sums
        dim3 grid((unsigned)(p.LN / KLC_COLS));
        if (sr_t == 1) hipLaunchKernelGGL(skinny_kl_cols_kernel<1>, grid, dim3(KLC_THREADS), 0, stream, p);
        else hipLaunchKernelGGL(skinny_kl_cols_kernel<2>, grid, dim3(KLC_THREADS), 0, stream, p);
    } else if (l_is_kl) {
        const unsigned lblocks = (unsigned)((p.LN + 255) / 256);
        // split k until ~4 blocks per CU are in flight, keeping at least 64 k per block
        int ksplit = (int)(1024 / ((long)lblocks * batch));
        const int kmax = (p.K + 63) / 64;
        if (ksplit > kmax) ksplit = kmax;
        if (ksplit < 1) ksplit = 1;
        if (ksplit > 65535) ksplit = 65535;
        p.kslice = ((p.K + ksplit - 1) / ksplit + 3) / 4 * 4;
        p.ksplit = (p.K + p.kslice - 1) / p.kslice;
        if (p.ksplit > 1) {
            rc = workspace_alloc(reinterpret_cast<void**>(&partial), sizeof(float) * batch * p.ksplit * p.SR * p.LN, stream);
            if (rc) return rc;
            p.partial = partial;
        }
        dim3 grid(lblocks, (unsigned)p.ksplit, batch);
        switch (sr_t) {
            case 1: hipLaunchKernelGGL(skinny_kl_kernel<1>, grid, dim3(256), 0, stream, p); break;
            case 2: hipLaunchKernelGGL(skinny_kl_kernel<2>, grid, dim3(256), 0, stream, p); break;
            case 4: hipLaunchKernelGGL(skinny_kl_kernel<4>, grid, dim3(256), 0, stream, p); break;
            default: hipLaunchKernelGGL(skinny_kl_kernel<8>, grid, dim3(256), 0, stream, p); break;
        }
        if (p.ksplit > 1) {
            dim3 g2((unsigned)(((long)p.SR * p.LN + 63) / 64), 1, batch);
            hipLaunchKernelGGL(skinny_reduce_kernel, g2, dim3(256), 0, stream, p);
        }
    } else {
        dim3 grid((unsigned)((p.LN + 15) / 16), 1, batch);
        if (grid.x > 0x7fffffffu / 2) return set_error(NZHIP_E_UNSUPPORTED, "nzhip_gemm: long extent too large");
        switch (sr_t) {
            case 1: hipLaunchKernelGGL(skinny_lk_kernel<1>, grid, dim3(256), 0, stream, p); break;
            case 2: hipLaunchKernelGGL(skinny_lk_kernel<2>, grid, dim3(256), 0, stream, p); break;
            case 4: hipLaunchKernelGGL(skinny_lk_kernel<4>, grid, dim3(256), 0, stream, p); break;
            default: hipLaunchKernelGGL(skinny_lk_kernel<8>, grid, dim3(256), 0, stream, p); break;
        }
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) rc = set_hip_error(e, "skinny GEMM kernel launch");
    if (partial) {
        int rc2 = workspace_free(partial, stream);
        if (!rc) rc = rc2;
    }
    return rc;
}

// ---- thin products: a short contraction and one narrow extent --------------------------------------
// K <= 32 and min(M, N) <= 16 with the other extent long (a Linear layer with a huge fan-in seen from its
// backward: dW[16 x 260100] = dy[16 x batch] x^T, dx[260100 x batch] = W^T dy). The output and the long
// operand are streamed once; a 128 x 128 MFMA tile would be empty to seven eighths. One lane owns one
// index l of the long extent and keeps the T <= 16 outputs of its row (column) in registers; the narrow
// operand sits in LDS, rounded, and is read as broadcasts. Every output is one chain of FMAs over
// ascending k of fp16-rounded operands: the k-ascending fp32 sum of the CPU restatement, bit for bit.
struct ThinArgs {
    const float* X;         // long operand: element (l, k) at X[l * x_sl + k * x_sk]
    const float* S;         // narrow operand: element (t, k) at S[t * s_st + k * s_sk]
    float* C;               // element (l, t) at C[l * c_sl + t * c_st]
    const float* bias;      // element (l, t) at bias[l * b_sl + t * b_st], or null
    long L, x_sl, x_sk, s_st, s_sk, c_sl, c_st, b_sl, b_st;
    int T, K, relu;
};

constexpr int THIN_MAX_T = 16, THIN_MAX_K = 32;

template <int T_T>
__global__ __launch_bounds__(256) void gemm_thin_kernel(const ThinArgs p) {
    __shared__ float s_lds[THIN_MAX_T * THIN_MAX_K];             // [t][k], rounded to fp16
    for (int i = threadIdx.x; i < T_T * p.K; i += 256) {
        const int t = i / p.K, k = i % p.K;
        s_lds[t * THIN_MAX_K + k] = t < p.T ? (float)(_Float16)p.S[t * p.s_st + k * p.s_sk] : 0.f;
    }
    __syncthreads();
    const long l = (long)blockIdx.x * 256 + threadIdx.x;
    if (l >= p.L) return;
    float acc[T_T];
#pragma unroll
    for (int t = 0; t < T_T; t++) acc[t] = 0.f;
    const float* xr = p.X + l * p.x_sl;
    for (int k = 0; k < p.K; k++) {
        const float x = (float)(_Float16)xr[k * p.x_sk];
#pragma unroll
        for (int t = 0; t < T_T; t++) acc[t] = __builtin_fmaf(x, s_lds[t * THIN_MAX_K + k], acc[t]);
    }
#pragma unroll
    for (int t = 0; t < T_T; t++) {
        if (t >= p.T) break;
        float v = acc[t];
        if (p.bias) v += p.bias[l * p.b_sl + t * p.b_st];
        if (p.relu) v = v > 0.f ? v : 0.f;
        p.C[l * p.c_sl + t * p.c_st] = v;
    }
}

bool gemm_thin_applicable(const nzhip_gemm_desc& d) {
    static const char* env = getenv("NZHIP_THIN");               // benchmarking only: 0 switches the route off
    if (env && atoi(env) == 0) return false;
    const int64_t lo = d.M < d.N ? d.M : d.N, hi = d.M < d.N ? d.N : d.M;
    return d.batch_n * d.batch_c == 1 && d.K >= 1 && d.K <= THIN_MAX_K && lo <= THIN_MAX_T && hi >= 2048;
}

int gemm_thin_dispatch(const nzhip_gemm_desc& d, hipStream_t stream) {
    ThinArgs p;
    const bool long_n = d.N >= d.M;
    // strides of A(m, k) and B(k, n) as stored
    const long a_sm = d.a_layout == NZHIP_LAYOUT_ROW ? d.lda : 1, a_sk = d.a_layout == NZHIP_LAYOUT_ROW ? 1 : d.lda;
    const long b_sk = d.b_layout == NZHIP_LAYOUT_ROW ? d.ldb : 1, b_sn = d.b_layout == NZHIP_LAYOUT_ROW ? 1 : d.ldb;
    if (long_n) {
        p.X = d.B; p.x_sl = b_sn; p.x_sk = b_sk;
        p.S = d.A; p.s_st = a_sm; p.s_sk = a_sk;
        p.L = d.N; p.T = (int)d.M;
        p.c_sl = 1; p.c_st = d.ldc;
        p.b_sl = d.bias_stride_col; p.b_st = d.bias_stride_row;
    } else {
        p.X = d.A; p.x_sl = a_sm; p.x_sk = a_sk;
        p.S = d.B; p.s_st = b_sn; p.s_sk = b_sk;
        p.L = d.M; p.T = (int)d.N;
        p.c_sl = d.ldc; p.c_st = 1;
        p.b_sl = d.bias_stride_row; p.b_st = d.bias_stride_col;
    }
    p.C = d.C; p.bias = d.bias; p.K = (int)d.K; p.relu = d.activation == NZHIP_ACT_RELU;
    const long blocks = (p.L + 255) / 256;
    if (blocks > 0x7fffffffL) return set_error(NZHIP_E_UNSUPPORTED, "nzhip_gemm: long extent too large");
    dim3 grid((unsigned)blocks);
    if (p.T <= 4) hipLaunchKernelGGL(gemm_thin_kernel<4>, grid, dim3(256), 0, stream, p);
    else if (p.T <= 8) hipLaunchKernelGGL(gemm_thin_kernel<8>, grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL(gemm_thin_kernel<16>, grid, dim3(256), 0, stream, p);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? NZHIP_OK : set_hip_error(e, "thin GEMM kernel launch");
}

}  // namespace nzhip
