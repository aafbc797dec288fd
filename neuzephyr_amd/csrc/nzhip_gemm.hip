// fp32-in / fp16-MFMA / fp32-accumulate GEMM for gfx950 (MI355X).
//
// One kernel family replaces the reference's Padding -> GeneralMatrixMulTensorKernel
// -> Cutting pipeline (src/OperationKernels.cu:821-871) and its per-(n,c) launch
// loops (:914-1026):
//   * operands are read as fp32 straight from the caller's buffers, rounded to
//     fp16 (v_cvt_pk_f16_f32, round-to-nearest-even) on the way into LDS;
//   * v_mfma_f32_32x32x16_f16 with fp32 accumulators;
//   * two LDS stages (one barrier per k tile), rows padded by 16 B so that the
//     128-bit fragment reads and the staging writes hit distinct banks;
//   * edges are predicated (zero fill on load, masked store) -- no padded copies;
//   * batch (n,c), broadcast strides, bias and ReLU are handled in-kernel.
#include <hip/hip_runtime.h>

#include <cstdlib>

#include "nzhip_internal.h"

namespace nzhip {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));

struct GemmKernelArgs {
    const float* A;
    const float* B;
    float* C;
    const float* bias;
    int M, N, K;
    long lda, ldb, ldc;
    int batch_c;                      // inner batch extent
    int batch;                        // batch_n * batch_c (the grid holds tiles_m * tiles_n * batch workgroups)
    long a_sn, a_sc, b_sn, b_sc, c_sn, c_sc, bias_sn, bias_sc;
    long bias_sm, bias_sk;            // bias row / column strides
    int relu;
    int tiles_m, tiles_n;
    int group_m;                      // tile rows per rasterisation group
    int k_total;                      // > 0: member j of the inner batch contracts min(K, k_total - j*K) (split-k chunks)
    int c_vec;                        // 16-byte stores to C are legal (alignment, ldc and N multiples of 4)
};

// Physical LDS row of logical tile row r. A wave owns TR = 32*FR logical rows; its MFMA
// block f (0..FR-1) takes the rows r with (r % TR) % FR == f, so that (a) the 32 rows one
// fragment read touches are consecutive in LDS and (b) each lane ends up holding FR
// consecutive output columns, which makes the C store a vector store.
template <int TR, int FR>
__device__ __forceinline__ int phys_row(int r) {
    const int w = r / TR, l = r % TR;
    return (w * FR + (l % FR)) * 32 + l / FR;
}

// ---- operand staging: global fp32 -> registers -> fp16 in LDS ----------------------------
// KCONTIG: the operand is stored with k contiguous (A row-major MxK, or B given as NxK).
// FULL: the tile lies wholly inside the operand and K is a multiple of BK, so no predicate is
// evaluated. Otherwise loads are predicated WITHOUT branches: an out-of-range lane reads the
// operand's first element (always mapped) and the value is replaced by zero afterwards.
template <int BR, int BK, int NT, int TR, int FR, int ROWB, bool VEC, bool FULL>
struct StageKContig {
    static constexpr int F4_PER_ROW = BK / 4;
    static constexpr int ROWS_PER_PASS = NT / F4_PER_ROW;
    static constexpr int PASSES = BR / ROWS_PER_PASS;
    static_assert(BR % ROWS_PER_PASS == 0 && PASSES >= 1, "tile/thread mismatch");
    floatx4 regs[PASSES];

    __device__ __forceinline__ void load(const float* __restrict__ X, long ldx, int row_base, int R, int k_base,
                                         int K, int tid) {
        const int k4 = tid % F4_PER_ROW, r0 = tid / F4_PER_ROW;
        const int gk = k_base + k4 * 4;
#pragma unroll
        for (int p = 0; p < PASSES; p++) {
            const int gr = row_base + r0 + p * ROWS_PER_PASS;
            const float* src = X + (long)gr * ldx + gk;
            if constexpr (FULL) {
                regs[p] = *reinterpret_cast<const floatx4*>(src);
            } else if constexpr (VEC) {
                const bool ok = gr < R && gk < K;
                const floatx4 v = *reinterpret_cast<const floatx4*>(ok ? src : X);
                const floatx4 z = {0.f, 0.f, 0.f, 0.f};
                regs[p] = ok ? v : z;
            } else {
                floatx4 v;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const bool ok = gr < R && gk + e < K;
                    const float x = *(ok ? src + e : X);
                    v[e] = ok ? x : 0.f;
                }
                regs[p] = v;
            }
        }
    }

    __device__ __forceinline__ void store(char* lds, int tid) const {
        const int k4 = tid % F4_PER_ROW, r0 = tid / F4_PER_ROW;
#pragma unroll
        for (int p = 0; p < PASSES; p++) {
            const int r = r0 + p * ROWS_PER_PASS;
            half4_t h;
            h[0] = (_Float16)regs[p][0];
            h[1] = (_Float16)regs[p][1];
            h[2] = (_Float16)regs[p][2];
            h[3] = (_Float16)regs[p][3];
            *reinterpret_cast<half4_t*>(lds + phys_row<TR, FR>(r) * ROWB + k4 * 8) = h;
        }
    }
};

// RCONTIG: the operand is stored with the tile dimension contiguous (B row-major KxN, or
// A given as KxM). Each thread takes 4 neighbouring tile rows over KPT consecutive k and
// transposes them in registers, so LDS still holds k-contiguous rows.
template <int BR, int BK, int NT, int TR, int FR, int ROWB, bool VEC, bool FULL>
struct StageRContig {
    static constexpr int F4_PER_KROW = BR / 4;
    static constexpr int KGROUPS = NT / F4_PER_KROW;
    static constexpr int KPT = BK / KGROUPS;
    static_assert(NT % F4_PER_KROW == 0 && KGROUPS >= 1 && BK % KGROUPS == 0, "tile/thread mismatch");
    static_assert(KPT == 2 || KPT == 4 || KPT == 8, "k per thread must be 2, 4 or 8");
    floatx4 regs[KPT];

    __device__ __forceinline__ void load(const float* __restrict__ X, long ldx, int row_base, int R, int k_base,
                                         int K, int tid) {
        const int r4 = tid % F4_PER_KROW, kg = tid / F4_PER_KROW;
        const int gr = row_base + r4 * 4;
#pragma unroll
        for (int q = 0; q < KPT; q++) {
            const int gk = k_base + kg * KPT + q;
            const float* src = X + (long)gk * ldx + gr;
            if constexpr (FULL) {
                regs[q] = *reinterpret_cast<const floatx4*>(src);
            } else if constexpr (VEC) {
                const bool ok = gk < K && gr < R;
                const floatx4 v = *reinterpret_cast<const floatx4*>(ok ? src : X);
                const floatx4 z = {0.f, 0.f, 0.f, 0.f};
                regs[q] = ok ? v : z;
            } else {
                floatx4 v;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const bool ok = gk < K && gr + e < R;
                    const float x = *(ok ? src + e : X);
                    v[e] = ok ? x : 0.f;
                }
                regs[q] = v;
            }
        }
    }

    __device__ __forceinline__ void store(char* lds, int tid) const {
        const int r4 = tid % F4_PER_KROW, kg = tid / F4_PER_KROW;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            char* dst = lds + phys_row<TR, FR>(r4 * 4 + e) * ROWB + kg * KPT * 2;
            if constexpr (KPT == 8) {
                half8_t h;
#pragma unroll
                for (int q = 0; q < 8; q++) h[q] = (_Float16)regs[q][e];
                *reinterpret_cast<half8_t*>(dst) = h;
            } else if constexpr (KPT == 4) {
                half4_t h;
#pragma unroll
                for (int q = 0; q < 4; q++) h[q] = (_Float16)regs[q][e];
                *reinterpret_cast<half4_t*>(dst) = h;
            } else {
                half2_t h;
                h[0] = (_Float16)regs[0][e];
                h[1] = (_Float16)regs[1][e];
                *reinterpret_cast<half2_t*>(dst) = h;
            }
        }
    }
};

template <bool RCONTIG, int BR, int BK, int NT, int TR, int FR, int ROWB, bool VEC, bool FULL>
struct StageSelect {
    using type = StageKContig<BR, BK, NT, TR, FR, ROWB, VEC, FULL>;
};
template <int BR, int BK, int NT, int TR, int FR, int ROWB, bool VEC, bool FULL>
struct StageSelect<true, BR, BK, NT, TR, FR, ROWB, VEC, FULL> {
    using type = StageRContig<BR, BK, NT, TR, FR, ROWB, VEC, FULL>;
};

// ---- the kernel ----------------------------------------------------------------------------
// BM x BN x BK workgroup tile, WM x WN waves, each wave a (BM/WM) x (BN/WN) tile of 32x32 MFMA
// blocks.  A_TRANS: A given as KxM.  B_TRANS: B given as NxK.  VEC: 16-byte global accesses
// are legal for both operands (alignment and extents checked on the host).  FULL: M, N and K
// are multiples of BM, BN and BK (implies VEC), so loads and stores carry no predicates.
template <int BM, int BN, int BK, int WM, int WN, bool A_TRANS, bool B_TRANS, bool VEC, bool FULL>
__global__ __launch_bounds__(WM* WN * 64) void gemm_f16mfma_kernel(const GemmKernelArgs p) {
    constexpr int NT = WM * WN * 64;
    constexpr int TM = BM / WM, TN = BN / WN;
    constexpr int FM = TM / 32, FN = TN / 32;
    constexpr int ROWB = BK * 2 + 16;                     // LDS row pitch in bytes
    constexpr int A_BYTES = BM * ROWB, B_BYTES = BN * ROWB;
    constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
    static_assert(TM % 32 == 0 && TN % 32 == 0 && BK % 16 == 0, "tile shape");

    extern __shared__ __attribute__((aligned(16))) char lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int li = lane & 31, lh = lane >> 5;

    // ---- which tile: spread consecutive ids over the 8 XCDs, then walk column-major inside
    // groups of group_m tile rows so that the workgroups resident on one XCD share A rows
    // and B columns in that XCD's L2.
    // The grid is one-dimensional over (batch member, tile), member-major: each XCD gets one
    // contiguous eighth of that list, so all tiles of a member with few tiles run on the same XCD
    // and its operands come from HBM once.
    const int total = p.tiles_m * p.tiles_n;
    int lin = blockIdx.x;
    {
        const int units = total * p.batch;
        const int xcd = lin & 7, q = lin >> 3;
        const int per = units >> 3, rem = units & 7;
        lin = xcd * per + (xcd < rem ? xcd : rem) + q;
    }
    const int member = lin / total;
    lin -= member * total;
    const int group_sz = p.group_m * p.tiles_n;
    const int group = lin / group_sz;
    const int first_m = group * p.group_m;
    const int rows_in_group = (p.tiles_m - first_m) < p.group_m ? (p.tiles_m - first_m) : p.group_m;
    const int tile_m = first_m + (lin % group_sz) % rows_in_group;
    const int tile_n = (lin % group_sz) / rows_in_group;
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    const int bi = member / p.batch_c, bj = member % p.batch_c;
    const float* __restrict__ A = p.A + bi * p.a_sn + bj * p.a_sc;
    const float* __restrict__ B = p.B + bi * p.b_sn + bj * p.b_sc;
    float* __restrict__ C = p.C + bi * p.c_sn + bj * p.c_sc;

    using StageA = typename StageSelect<A_TRANS, BM, BK, NT, TM, FM, ROWB, VEC, FULL>::type;
    using StageB = typename StageSelect<!B_TRANS, BN, BK, NT, TN, FN, ROWB, VEC, FULL>::type;
    // With 128 or fewer accumulator registers per lane (128x128 tiles, or 256x256 tiles on eight waves)
    // there is room for a second staging set per operand: the tile two k steps ahead is requested
    // while the current one is multiplied, so a request has two MFMA phases to land before it is
    // converted into LDS. The 256x256 tile on four waves (256 accumulator registers per lane) stages
    // one tile ahead.
    constexpr bool TWO_AHEAD = BM * BN <= 128 * 128 || WM * WN >= 8;
    StageA sa0, sa1;
    StageB sb0, sb1;

    floatx16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    // the last chunk of a split contraction may be shorter than the others
    const int K = (p.k_total > 0 && p.k_total - bj * p.K < p.K) ? p.k_total - bj * p.K : p.K;
    const int nk = (K + BK - 1) / BK;

    // LDS-only barrier: waits for this wave's LDS traffic, not for the global requests in flight
    auto lds_barrier = []() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
    // Requests past the last tile repeat the last tile (results unused): the number of requests
    // per step is the same on every path, so each wait names exactly the set it needs.
    auto request = [&](StageA& ra, StageB& rb, int kt) {
        const int kc = kt < nk ? kt : nk - 1;
        ra.load(A, p.lda, m0, p.M, kc * BK, K, tid);
        rb.load(B, p.ldb, n0, p.N, kc * BK, K, tid);
    };
    auto multiply = [&](const char* cur) {
        const char* la = cur + ((wm * FM) * 32 + li) * ROWB + lh * 16;
        const char* lb = cur + A_BYTES + ((wn * FN) * 32 + li) * ROWB + lh * 16;
#pragma unroll
        for (int ks = 0; ks < BK / 16; ks++) {
            half8_t af[FM], bf[FN];
#pragma unroll
            for (int i = 0; i < FM; i++) af[i] = *reinterpret_cast<const half8_t*>(la + i * 32 * ROWB + ks * 32);
#pragma unroll
            for (int j = 0; j < FN; j++) bf[j] = *reinterpret_cast<const half8_t*>(lb + j * 32 * ROWB + ks * 32);
#pragma unroll
            for (int i = 0; i < FM; i++)
#pragma unroll
                for (int j = 0; j < FN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
    };
    if constexpr (TWO_AHEAD) {
        // one k step: tile kt is in LDS stage `cur`; `ra/rb` held it and are free again; `qa/qb`
        // hold tile kt + 1. Steps come in pairs; with an odd tile count the last step only moves
        // data (requests and stores are issued on every path, the MFMAs are skipped).
        auto step = [&](int kt, char* cur, char* nxt, StageA& ra, StageB& rb, StageA& qa, StageB& qb) {
            request(ra, rb, kt + 2);
            if (kt < nk) multiply(cur);
            qa.store(nxt, tid);                               // tile kt + 1 (a repeat of the last tile past the end)
            qb.store(nxt + A_BYTES, tid);
            lds_barrier();
        };
        request(sa0, sb0, 0);
        request(sa1, sb1, 1);
        sa0.store(lds, tid);
        sb0.store(lds + A_BYTES, tid);
        lds_barrier();
        char* st0 = lds;
        char* st1 = lds + STAGE_BYTES;
        for (int kt = 0; kt < nk; kt += 2) {
            step(kt, st0, st1, sa0, sb0, sa1, sb1);
            step(kt + 1, st1, st0, sa1, sb1, sa0, sb0);
        }
        // the requests issued for tiles past the end are still in flight: take delivery before
        // the registers are reused by the epilogue
        __builtin_amdgcn_s_waitcnt(0x0070 | 0x0F00);
    } else {
        sa0.load(A, p.lda, m0, p.M, 0, K, tid);
        sb0.load(B, p.ldb, n0, p.N, 0, K, tid);
        sa0.store(lds, tid);
        sb0.store(lds + A_BYTES, tid);
        __syncthreads();
        for (int kt = 0; kt < nk; kt++) {
            char* cur = lds + (kt & 1) * STAGE_BYTES;
            char* nxt = lds + ((kt + 1) & 1) * STAGE_BYTES;
            const bool more = kt + 1 < nk;
            if (more) {
                sa0.load(A, p.lda, m0, p.M, (kt + 1) * BK, K, tid);
                sb0.load(B, p.ldb, n0, p.N, (kt + 1) * BK, K, tid);
            }
            multiply(cur);
            if (more) {
                sa0.store(nxt, tid);
                sb0.store(nxt + A_BYTES, tid);
            }
            __syncthreads();
        }
    }

    // ---- epilogue: bias, activation, predicated (vector when legal) store ------------------
    // Bias values are fetched in batches (all of a 32-row block at once, or once per lane when
    // the bias does not vary along rows) so the stores never wait on one load each.
    const float* bias = p.bias ? p.bias + bi * p.bias_sn + bj * p.bias_sc : nullptr;
    const int gn = n0 + wn * TN + li * FN;                // first of this lane's FN columns
    const bool vec_store = FULL || (VEC && p.c_vec && (FN == 2 || FN == 4) && (gn + FN <= p.N));
    float bcol[FN];
    const bool bias_rowless = bias && p.bias_sm == 0;
#pragma unroll
    for (int j = 0; j < FN; j++) bcol[j] = (bias_rowless && gn + j < p.N) ? bias[(long)(gn + j) * p.bias_sk] : 0.f;
    // A bias that varies along rows (a bias matrix, C itself when a gradient is accumulated in place) is requested half
    // a block (8 rows) ahead of the stores that need it: a load issued after stores is not counted as returned before
    // those stores are acknowledged, so requesting a block after storing the one before made every block wait for
    // its predecessor. 16- or 8-byte loads when the bias rows are contiguous and aligned like the rows of C.
    const bool bias_rows = bias && !bias_rowless;
    const bool bias_vec = bias_rows && (FN == 2 || FN == 4) && p.bias_sk == 1 && (p.bias_sm & (FN - 1)) == 0 &&
                          (reinterpret_cast<uintptr_t>(bias) & (FN * 4 - 1)) == 0 && gn + FN <= p.N;
    float bvs[2][8][FN];
    auto bias_request = [&](float (&bv)[8][FN], const int i, const int h) {
#pragma unroll
        for (int r8 = 0; r8 < 8; r8++) {
            const int r = h * 8 + r8;
            const int gm = m0 + wm * TM + ((r >> 2) * 8 + lh * 4 + (r & 3)) * FM + i;
            const float* bp = bias + (long)(gm < p.M ? gm : 0) * p.bias_sm;
            if (bias_vec) {
                if constexpr (FN == 4) {
                    const floatx4 v = *reinterpret_cast<const floatx4*>(bp + gn);
#pragma unroll
                    for (int e = 0; e < 4; e++) bv[r8][e] = v[e];
                } else if constexpr (FN == 2) {
                    const floatx2 v = *reinterpret_cast<const floatx2*>(bp + gn);
                    bv[r8][0] = v[0];
                    bv[r8][1] = v[1];
                }
            } else {
#pragma unroll
                for (int j = 0; j < FN; j++) bv[r8][j] = bp[gn + j < p.N ? (long)(gn + j) * p.bias_sk : 0];
            }
        }
    };
    if (bias_rows) bias_request(bvs[0], 0, 0);
#pragma unroll
    for (int i = 0; i < FM; i++) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            if (bias_rows && (r & 7) == 0 && i * 2 + (r >> 3) + 1 < 2 * FM)
                bias_request(bvs[(i * 2 + (r >> 3) + 1) & 1], (i * 2 + (r >> 3) + 1) >> 1, (i * 2 + (r >> 3) + 1) & 1);
            const int im = (r >> 2) * 8 + lh * 4 + (r & 3);
            const int gm = m0 + wm * TM + im * FM + i;
            if (!FULL && gm >= p.M) continue;
            float v[FN];
#pragma unroll
            for (int j = 0; j < FN; j++) {
                float x = acc[i][j][r] + (bias_rows ? bvs[(i * 2 + (r >> 3)) & 1][r & 7][j] : bcol[j]);
                if (p.relu) x = x > 0.f ? x : 0.f;
                v[j] = x;
            }
            float* dst = C + (long)gm * p.ldc + gn;
            if (vec_store) {
                if constexpr (FN == 4) {
                    floatx4 o = {v[0], v[1], v[2], v[3]};
                    *reinterpret_cast<floatx4*>(dst) = o;
                } else if constexpr (FN == 2) {
                    floatx2 o = {v[0], v[1]};
                    *reinterpret_cast<floatx2*>(dst) = o;
                } else {
                    dst[0] = v[0];
                }
            } else {
#pragma unroll
                for (int j = 0; j < FN; j++)
                    if (gn + j < p.N) dst[j] = v[j];
            }
        }
    }
}

// ---- host-side selection -------------------------------------------------------------------
template <int BM, int BN, int BK, int WM, int WN>
static int launch_cfg(const GemmKernelArgs& a, bool a_trans, bool b_trans, bool vec, int batch, hipStream_t s) {
    const bool full = vec && a.c_vec && a.M % BM == 0 && a.N % BN == 0 && a.K % BK == 0 && (a.k_total <= 0 || a.k_total % a.K == 0);
    constexpr int ROWB = BK * 2 + 16;
    constexpr size_t lds_bytes = 2 * (size_t)(BM + BN) * ROWB;
    dim3 grid((unsigned)((int64_t)a.tiles_m * a.tiles_n * batch), 1, 1), block(WM * WN * 64, 1, 1);
#define NZHIP_LAUNCH(AT, BT, V, F)                                                                       \
    do {                                                                                                 \
        auto kfn = gemm_f16mfma_kernel<BM, BN, BK, WM, WN, AT, BT, V, F>;                                \
        if (int lrc = ensure_dynamic_lds(reinterpret_cast<const void*>(kfn), (int)lds_bytes,             \
                                         "hipFuncSetAttribute(gemm)"))                                   \
            return lrc;                                                                                  \
        hipLaunchKernelGGL(kfn, grid, block, lds_bytes, s, a);                                           \
    } while (0)
    if (full) {
        if (!a_trans && !b_trans) NZHIP_LAUNCH(false, false, true, true);
        else if (!a_trans && b_trans) NZHIP_LAUNCH(false, true, true, true);
        else if (a_trans && !b_trans) NZHIP_LAUNCH(true, false, true, true);
        else NZHIP_LAUNCH(true, true, true, true);
    } else if (vec) {
        if (!a_trans && !b_trans) NZHIP_LAUNCH(false, false, true, false);
        else if (!a_trans && b_trans) NZHIP_LAUNCH(false, true, true, false);
        else if (a_trans && !b_trans) NZHIP_LAUNCH(true, false, true, false);
        else NZHIP_LAUNCH(true, true, true, false);
    } else {
        if (!a_trans && !b_trans) NZHIP_LAUNCH(false, false, false, false);
        else if (!a_trans && b_trans) NZHIP_LAUNCH(false, true, false, false);
        else if (a_trans && !b_trans) NZHIP_LAUNCH(true, false, false, false);
        else NZHIP_LAUNCH(true, true, false, false);
    }
#undef NZHIP_LAUNCH
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return set_hip_error(e, "gemm kernel launch");
    return NZHIP_OK;
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// 16-byte accesses are legal when every row start is 16-byte aligned and the contiguous extent is
// a multiple of 4, for every batch member: the operands decide which kernel instance loads them,
// C only whether the epilogue may use vector stores.
bool gemm_operand_vec_legal(const float* X, int64_t ld, int64_t contig, int64_t stride_n, int64_t stride_c) {
    auto ok4 = [](int64_t v) { return (v & 3) == 0; };
    return aligned16(X) && ok4(ld) && ok4(contig) && ok4(stride_n) && ok4(stride_c);
}

// padded: bit 0 / bit 1 = the rows of A / B are readable up to the next multiple of 4 elements and hold
// zeros there (the library's own padded copies), so their contiguous extent need not be a multiple of 4
bool gemm_operands_vec_legal(const nzhip_gemm_desc& d, int padded) {
    const bool a_trans = d.a_layout == NZHIP_LAYOUT_TRANS, b_trans = d.b_layout == NZHIP_LAYOUT_TRANS;
    return gemm_operand_vec_legal(d.A, d.lda, (padded & 1) ? 0 : (a_trans ? d.M : d.K), d.a_stride_n, d.a_stride_c) &&
           gemm_operand_vec_legal(d.B, d.ldb, (padded & 2) ? 0 : (b_trans ? d.K : d.N), d.b_stride_n, d.b_stride_c);
}

bool gemm_c_vec_legal(const nzhip_gemm_desc& d) {
    return gemm_operand_vec_legal(d.C, d.ldc, d.N, d.c_stride_n, d.c_stride_c);
}

bool gemm_vec_legal(const nzhip_gemm_desc& d) { return gemm_operands_vec_legal(d, 0) && gemm_c_vec_legal(d); }

// ---- tile and split choice for products that do not fill the device -------------------------------
// The fused kernel's k loop is bound by the rate at which one CU takes fp32 tiles in through its L1
// (about 50 GB/s per CU with 16-byte loads, 36 GB/s when they carry predicates, 9 GB/s element by element), so the time of a launch is
// the bytes the busiest CU streams: rounds of workgroups x (tile rows + tile columns, as far as the
// operands reach) x chunk length x 4 bytes. 64 x 64 tiles stream twice the bytes of 128 x 128 tiles in total but put four times
// as many CUs to work (1024^3: 23.6 us -> 14.2 us); a split contraction adds a pass over the partial sums.
struct FusedCostInput {
    int64_t M, N, K, members;       // members: batch_n * batch_c of the product as given
    double cus;
    bool vec, c_vec;
};

static double fused_cost_us(const FusedCostInput& q, int tile, int64_t parts, int64_t Kc) {
    const int64_t tiles = ((q.M + tile - 1) / tile) * ((q.N + tile - 1) / tile) * q.members * parts;
    const double rounds = (double)((tiles + (int64_t)q.cus - 1) / (int64_t)q.cus);
    const bool full = q.vec && q.c_vec && q.M % tile == 0 && q.N % tile == 0 && Kc % 32 == 0 && q.K % 32 == 0;   // unpredicated instance
    // rows past the operand's extent are predicated off, not loaded: a narrow operand costs what it has
    const double rows = (double)(q.M < tile ? q.M : tile) + (double)(q.N < tile ? q.N : tile);
    // two or more workgroups on a CU overlap their waits: the CU takes in up to 1.3 x what one workgroup draws
    // (16 x 8192 x 8192: 50 us in eight chunks, two workgroups per CU, against 57 us in four)
    const double per_cu = (double)tiles / q.cus;
    const double overlap = per_cu >= 2.0 ? 1.3 : per_cu > 1.0 ? 1.0 + 0.3 * (per_cu - 1.0) : 1.0;
    const double stream = rounds * rows * (double)Kc * 4.0 / ((full ? 50e3 : q.vec ? 36e3 : 9e3) * overlap);   // bytes / (bytes per us)
    const double out = (double)q.M * q.N * q.members * 4.0;
    const double reduce = parts > 1 ? 6.0 + (double)(parts + 1) * out / 3e6 : 0.0;
    // what a workgroup spends outside its k loop (first requests, predicated epilogue): 17 x 33 x 15 takes 10 us with a
    // 128 x 128 tile and 5 us with a 64 x 64 tile; rounds that share a CU pay it side by side
    const double ends = (tile == 64 ? 1.5 : 4.0) * (rounds > 2.0 ? rounds / 2.0 : 1.0);
    return 3.0 + ends + stream + reduce;
}

static FusedCostInput fused_cost_input(const nzhip_gemm_desc& d, int padded) {
    return {d.M, d.N, d.K, d.batch_n * d.batch_c, (double)device_cu_count(), gemm_operands_vec_legal(d, padded), gemm_c_vec_legal(d)};
}

GemmPlan gemm_fused_plan(const nzhip_gemm_desc& d, int padded) {
    const FusedCostInput q = fused_cost_input(d, padded);
    GemmPlan best = {128, 1, d.K, 0.0};
    double best_cost = fused_cost_us(q, 128, 1, d.K);
    auto consider = [&](int tile, int64_t parts, int64_t Kc) {
        const double c = fused_cost_us(q, tile, parts, Kc);
        if (c < best_cost * 0.97) { best_cost = c; best = {tile, parts, Kc, 0.0}; }    // keep the plainer plan on a near tie
    };
    consider(64, 1, d.K);
    // a batch over n alone (batch_c == 1) can be split as well: the chunks take the c dimension of the launch
    if (d.batch_c == 1 && d.batch_n <= 65535 && d.K >= 512) {
        const bool narrow = d.M <= 64 || d.N <= 64;                // padded tiles: the k loop is shorter per byte
        const int64_t min_chunk = q.vec && !narrow ? 512 : 128;
        for (int64_t S = 2; S <= 1024 && S <= d.K / min_chunk; S += (S < 8 ? 1 : S / 4)) {   // about 25 candidates
            const int64_t Kc = ((d.K + S - 1) / S + 31) / 32 * 32;              // chunk length, whole 32-wide k tiles
            const int64_t parts = (d.K + Kc - 1) / Kc;                           // the last one may be shorter
            if (parts < 2) continue;
            consider(128, parts, Kc);
            consider(64, parts, Kc);
        }
    }
    best.cost_us = best_cost;
    return best;
}

bool gemm_small_tile(const nzhip_gemm_desc& d, int padded) {
    // called with the descriptor of the launch itself (split chunks are its inner batch)
    const FusedCostInput q = fused_cost_input(d, padded);
    return fused_cost_us(q, 64, 1, d.K) < 0.97 * fused_cost_us(q, 128, 1, d.K);
}

int gemm_mfma_dispatch(const nzhip_gemm_desc& d, hipStream_t stream, int force_tile, int64_t k_total, int padded) {
    GemmKernelArgs a;
    a.A = d.A;
    a.B = d.B;
    a.C = d.C;
    a.bias = d.bias;
    a.M = (int)d.M;
    a.N = (int)d.N;
    a.K = (int)d.K;
    a.lda = d.lda;
    a.ldb = d.ldb;
    a.ldc = d.ldc;
    a.batch_c = (int)d.batch_c;
    a.batch = (int)(d.batch_n * d.batch_c);
    a.a_sn = d.a_stride_n;
    a.a_sc = d.a_stride_c;
    a.b_sn = d.b_stride_n;
    a.b_sc = d.b_stride_c;
    a.c_sn = d.c_stride_n;
    a.c_sc = d.c_stride_c;
    a.bias_sn = d.bias_stride_n;
    a.bias_sc = d.bias_stride_c;
    a.bias_sm = d.bias_stride_row;
    a.bias_sk = d.bias_stride_col;
    a.relu = d.activation == NZHIP_ACT_RELU;
    a.k_total = (int)k_total;

    const bool a_trans = d.a_layout == NZHIP_LAYOUT_TRANS, b_trans = d.b_layout == NZHIP_LAYOUT_TRANS;
    const bool vec = gemm_operands_vec_legal(d, padded);
    a.c_vec = gemm_c_vec_legal(d);
    const int64_t batch = d.batch_n * d.batch_c;

    // Tile choice: 256x256 tiles need enough of them to fill the 256 CUs and pay only in their
    // unpredicated instance (5000x1000x5000: 379 us with predicated 256x256 tiles, 156 us with
    // 128x128 tiles).
    const int64_t t256 = ((d.M + 255) / 256) * ((d.N + 255) / 256) * batch;
    const bool whole256 = vec && a.c_vec && d.M % 256 == 0 && d.N % 256 == 0 && d.K % 32 == 0 && (k_total <= 0 || k_total % d.K == 0);
    static const char* tile_env = getenv("NZHIP_GEMM_TILE");         // 128 | 256: benchmarking only
    if (!force_tile && tile_env && (atoi(tile_env) == 128 || atoi(tile_env) == 256)) force_tile = atoi(tile_env);
    int tile = force_tile ? force_tile : (t256 >= 192 && whole256 ? 256 : gemm_small_tile(d, padded) ? 64 : 128);
    const int bm = tile, bn = tile;
    a.tiles_m = (int)((d.M + bm - 1) / bm);
    a.tiles_n = (int)((d.N + bn - 1) / bn);
    if ((int64_t)a.tiles_m * a.tiles_n * batch > 0x7fffffff)
        return set_error(NZHIP_E_UNSUPPORTED, "nzhip_gemm: more than 2^31 output tiles in one call");
    // rows per rasterisation group: with 32 workgroups resident per XCD aim at a 4x8 footprint
    a.group_m = 4;
    // 256x256 tiles run with 4 x 2 waves (two per SIMD, 128 accumulators each): that leaves registers for
    // the second staging set, and one wave converts while the other multiplies (batched 128 x 1024^3:
    // 0.63 ms with 2 x 2 waves, 0.55 ms with 4 x 2). NZHIP_GEMM_WAVES=4 selects 2 x 2 (benchmarking only).
    static const char* waves_env = getenv("NZHIP_GEMM_WAVES");
    if (tile == 256 && waves_env && atoi(waves_env) == 4)
        return launch_cfg<256, 256, 32, 2, 2>(a, a_trans, b_trans, vec, (int)batch, stream);
    if (tile == 256) return launch_cfg<256, 256, 32, 4, 2>(a, a_trans, b_trans, vec, (int)batch, stream);
    if (tile == 64) {
        // whole tiles: 64-wide k steps halve the number of barriers (1024^3: 14.2 -> 13.0 us); with predicates
        // the wider step only adds padding (1000 x 777 x 513: 22.0 -> 23.2 us)
        const bool whole = vec && a.c_vec && d.M % 64 == 0 && d.N % 64 == 0 && d.K % 64 == 0 && (k_total <= 0 || k_total % d.K == 0);
        if (whole) return launch_cfg<64, 64, 64, 2, 2>(a, a_trans, b_trans, vec, (int)batch, stream);
        return launch_cfg<64, 64, 32, 2, 2>(a, a_trans, b_trans, vec, (int)batch, stream);
    }
    return launch_cfg<128, 128, 32, 2, 2>(a, a_trans, b_trans, vec, (int)batch, stream);
}

}  // namespace nzhip
