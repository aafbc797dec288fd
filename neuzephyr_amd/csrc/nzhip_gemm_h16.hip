// Two-pass route for large products: round A and B to fp16 once into a pooled workspace
// (zero-padded to tile multiples, both with k contiguous), then run a pure-fp16 MFMA GEMM
// whose tiles travel global -> LDS directly (global_load_lds_dwordx4, no staging registers).
//
// Why two passes when the operands are large: with fp32 operands every workgroup has to pull
// 4 bytes per element through L2 and the vector memory path for every tile it touches
// (M/256 + N/256 times per element), and the 256x256 accumulator tile leaves a single wave
// per SIMD, i.e. nothing to hide the load latency behind. Rounding once (the same RNE
// conversion the reference's Padding kernel performs, src/OperationKernels.cu:846-860) halves
// the re-read traffic and frees the registers. Results are identical to the fused kernel's up
// to fp32 summation order.
#include <hip/hip_runtime.h>

#include <cstdlib>

#include "nzhip_internal.h"

namespace nzhip {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));

// ---- pass 1: rounding copies ---------------------------------------------------------------
// The workspace is NOT a row-major matrix. It is a sequence of 16 KiB blocks, one per
// (256-row block rb, 32-wide k tile kt), stored at block index rb * (Kp/32) + kt, and each
// block is the exact image the GEMM wants in LDS: physical row pr (see phys_row_of) at byte
// pr*64, chunk c (8 halfs) of that row at chunk position c ^ chunk_swizzle(pr). The GEMM's
// global->LDS copies are therefore plain contiguous 1 KiB reads, consecutive k tiles are
// consecutive 16 KiB blocks (no power-of-two row pitch, so all memory channels stay busy),
// and rows/columns beyond the operand are zero.
constexpr int CVT_ROWS = 256, CVT_K = 32, CVT_BLOCK_BYTES = CVT_ROWS * CVT_K * 2;

// Chunk swizzle of a 64-byte LDS row. A 128-bit LDS read is served 16 lanes per pass, and the passes
// are NOT lanes 0-15, 16-31, ...: lanes {0-3, 12-15, 20-23, 24-27} share one pass, {4-7, 8-11, 16-19,
// 28-31} the next (and the same again for lanes 32-63). In a 16x16x32 fragment read lane l takes
// chunk l>>4 of row l&15, so one pass mixes row quads 0 and 3 at chunk q with row quads 1 and 2 at
// chunk q^1. With f(quad) = -quad mod 4 the four (quad, chunk) pairs of every pass land on four
// different 16-byte bank groups; the plainer f(quad) = quad puts them on two, and every read takes
// 1.6 times as long (measured per instruction: 7.1 against 4.4 clocks).
__device__ __forceinline__ int chunk_swizzle(int row) { return (-(row >> 2)) & 3; }

// Physical LDS row of logical tile row r when a wave owns FR consecutive 32-row MFMA blocks of the
// 256-row tile (FR = 4: two waves along that dimension, FR = 2: four). The rows of a wave are
// interleaved over its blocks so that one lane ends up with FR adjacent rows / columns.
__device__ __forceinline__ int phys_row_of(int r, int fr, int blk) {
    const int tr = blk * fr, w = r / tr, l = r % tr;
    return (w * fr + (l % fr)) * blk + (l / fr);
}

// K_CONTIG: source element (r, k) at src[r*ld + k]; otherwise at src[k*ld + r].
struct CvtOperand {
    _Float16* dst;
    const float* src;
    int R;                      // rows of the operand (output rows for A, output columns for B)
    long ld, src_batch, dst_batch;
    int vec, fr;
};

template <bool K_CONTIG>
__device__ __forceinline__ void cvt_block(char* img, const CvtOperand& o, int K, int nkt, int blk, int kt, int rb, int member) {
    _Float16* dst = o.dst;
    const int R = o.R, vec = o.vec, fr = o.fr;
    const long ld = o.ld, dst_batch = o.dst_batch;
    const float* s = o.src + (long)member * o.src_batch;
    const int t = threadIdx.x;
    const int r0 = rb * CVT_ROWS, k0 = kt * CVT_K;
    if (K_CONTIG) {
        // 8 threads per row (one float4 each), 32 rows per pass
        const int k4 = t & 7, rr = t >> 3;
#pragma unroll
        for (int pass = 0; pass < 8; pass++) {
            const int lr = rr + pass * 32, r = r0 + lr, k = k0 + k4 * 4;
            floatx4 v = {0.f, 0.f, 0.f, 0.f};
            const float* q = s + (long)r * ld + k;
            if (r < R) {
                if (vec && k + 4 <= K) {
                    v = *reinterpret_cast<const floatx4*>(q);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (k + e < K) v[e] = q[e];
                }
            }
            half4_t h = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
            const int pr = phys_row_of(lr, fr, blk);
            const int pos = (k4 >> 1) ^ chunk_swizzle(pr);
            *reinterpret_cast<half4_t*>(img + pr * 64 + pos * 16 + (k4 & 1) * 8) = h;
        }
    } else {
        // 64 threads per k row (one float4 of 4 rows each), 4 k rows per pass
        const int r4 = t & 63, kk0 = t >> 6;
#pragma unroll
        for (int pass = 0; pass < 8; pass++) {
            const int kk = kk0 + pass * 4, k = k0 + kk, lr = r4 * 4, r = r0 + lr;
            floatx4 v = {0.f, 0.f, 0.f, 0.f};
            const float* q = s + (long)k * ld + r;
            if (k < K) {
                if (vec && r + 4 <= R) {
                    v = *reinterpret_cast<const floatx4*>(q);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (r + e < R) v[e] = q[e];
                }
            }
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int pr = phys_row_of(lr + e, fr, blk);
                const int pos = (kk >> 3) ^ chunk_swizzle(pr);
                *reinterpret_cast<_Float16*>(img + pr * 64 + pos * 16 + (kk & 7) * 2) = (_Float16)v[e];
            }
        }
    }
    __syncthreads();
    char* out = reinterpret_cast<char*>(dst + (long)member * dst_batch) + ((long)rb * nkt + kt) * CVT_BLOCK_BYTES;
#pragma unroll
    for (int pass = 0; pass < 4; pass++) {
        const int off = (pass * 256 + t) * 16;
        *reinterpret_cast<floatx4*>(out + off) = *reinterpret_cast<const floatx4*>(img + off);
    }
}

template <bool K_CONTIG>
__global__ __launch_bounds__(256) void cvt_block_kernel(CvtOperand o, int K, int nkt, int blk) {
    __shared__ __attribute__((aligned(16))) char img[CVT_BLOCK_BYTES];
    cvt_block<K_CONTIG>(img, o, K, nkt, blk, blockIdx.x, blockIdx.y, blockIdx.z);
}

// Both operands in one launch (the usual case: neither is batched differently from the other): row
// blocks [0, a_blocks) of the grid's y axis belong to A, the rest to B.
template <bool A_K_CONTIG, bool B_K_CONTIG>
__global__ __launch_bounds__(256) void cvt_pair_kernel(CvtOperand a, CvtOperand b, int a_blocks, int K, int nkt, int blk) {
    __shared__ __attribute__((aligned(16))) char img[CVT_BLOCK_BYTES];
    const int rb = blockIdx.y;
    if (rb < a_blocks)
        cvt_block<A_K_CONTIG>(img, a, K, nkt, blk, blockIdx.x, rb, blockIdx.z);
    else
        cvt_block<B_K_CONTIG>(img, b, K, nkt, blk, blockIdx.x, rb - a_blocks, blockIdx.z);
}

// ---- pass 2: fp16 GEMM -----------------------------------------------------------------------
struct H16Args {
    const _Float16* A;      // blocked image of A: [Mp/256][Kp/32] blocks of 16 KiB
    const _Float16* B;      // blocked image of B (rows = output columns): [Np/256][Kp/32] blocks
    float* C;
    const float* bias;
    int M, N, Kp;
    long ldc;
    int batch_c;
    int batch;                        // batch_n * batch_c
    long a_batch, b_batch;              // workspace strides per batch member (0 = shared operand)
    int a_bcast_n, a_bcast_c, b_bcast_n, b_bcast_c;   // 1 = operand is shared along that batch axis
    int a_cn;                           // extent of A's c axis in the workspace (for indexing)
    int b_cn;
    long c_sn, c_sc, bias_sn, bias_sc, bias_sm, bias_sk;
    int relu;
    int tiles_m, tiles_n, group_m;
};

// s_waitcnt on the vector-memory counter only (expcnt / lgkmcnt left at "don't wait").
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0070 | 0x0F00);
}
__device__ __forceinline__ void wait_lgkmcnt0() { __builtin_amdgcn_s_waitcnt(0xC07F); }   // lgkmcnt(0) only

// BM x BN x 32 tiles in an NSTAGE-deep LDS ring. One LDS row = 32 halfs = 64 bytes = 4 chunks of
// 16 bytes. LDS has 64 banks x 4 B, so a 256-byte bank row spans four tile rows; chunk c of row r
// is stored at chunk position  c ^ chunk_swizzle(r), which puts the 16 lanes that share one pass of a
// 128-bit fragment read on 16 different 16-byte bank groups.
template <int BM, int BN, int WM, int WN, int NSTAGE>
__global__ __launch_bounds__(WM* WN * 64, (BM < CVT_ROWS ? 2 : 1)) void gemm_h16_kernel(const H16Args p) {
    static_assert((BM == CVT_ROWS || BM * 2 == CVT_ROWS) && BN == CVT_ROWS, "must match the workspace block image");
    constexpr int BK = CVT_K, ROWB = 64;
    constexpr int NW = WM * WN;
    constexpr int TM = BM / WM, TN = BN / WN, FM = TM / 32, FN = TN / 32;
    constexpr int A_BYTES = BM * ROWB, B_BYTES = BN * ROWB, STAGE = A_BYTES + B_BYTES;
    constexpr int A_LOADS = BM / 16 / NW, B_LOADS = BN / 16 / NW;   // wave-wide 1 KiB loads (16 rows) per wave
    constexpr int LOADS = A_LOADS + B_LOADS;
    static_assert(BM % (16 * NW) == 0 && BN % (16 * NW) == 0, "tile/wave mismatch");
    static_assert((NSTAGE - 1) * LOADS < 64, "too many loads in flight for vmcnt");

    extern __shared__ __attribute__((aligned(1024))) char lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int li = lane & 31, lh = lane >> 5;

    // one-dimensional grid over (batch member, tile), member-major, one contiguous eighth per XCD
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
    const long a_idx = (long)(p.a_bcast_n ? 0 : bi) * p.a_cn + (p.a_bcast_c ? 0 : bj);
    const long b_idx = (long)(p.b_bcast_n ? 0 : bi) * p.b_cn + (p.b_bcast_c ? 0 : bj);
    const _Float16* __restrict__ A = p.A + a_idx * p.a_batch;
    const _Float16* __restrict__ B = p.B + b_idx * p.b_batch;
    float* __restrict__ C = p.C + bi * p.c_sn + bj * p.c_sc;

    // The workspace already holds the LDS image of every (row block, k tile): this wave's
    // share of a stage is A_LOADS + B_LOADS contiguous 1 KiB pieces, lane l taking bytes
    // [16 l, 16 l + 16) of each.
    const int nk = p.Kp / BK;
    // a BM = 128 tile is one half of a 256-row block of the image (its 128 physical rows are contiguous)
    constexpr int A_BLOCK = CVT_ROWS * ROWB, A_PER_BLOCK = CVT_ROWS / BM;
    const char* a_tile = reinterpret_cast<const char*>(A) + (long)(tile_m / A_PER_BLOCK) * nk * A_BLOCK +
                         (tile_m % A_PER_BLOCK) * A_BYTES + wave * A_LOADS * 1024 + lane * 16;
    const char* b_tile = reinterpret_cast<const char*>(B) + (long)tile_n * nk * B_BYTES + wave * B_LOADS * 1024 + lane * 16;

    // Request k tile kt into ring slot `stage`. Past the end the last tile is requested again
    // (into a slot nobody reads any more) so that the number of loads in flight, which the
    // vmcnt waits below count on, is the same in every iteration.
    auto issue_loads = [&](int kt, int stage) {
        const int kc = kt < nk ? kt : nk - 1;
        char* sa = lds + stage * STAGE + wave * A_LOADS * 1024;
        char* sb = lds + stage * STAGE + A_BYTES + wave * B_LOADS * 1024;
        const char* ak = a_tile + (long)kc * A_BLOCK;
        const char* bk = b_tile + (long)kc * B_BYTES;
#pragma unroll
        for (int j = 0; j < A_LOADS; j++)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(ak + j * 1024),
                                             (__attribute__((address_space(3))) void*)(sa + j * 1024), 16, 0, 0);
#pragma unroll
        for (int j = 0; j < B_LOADS; j++)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(bk + j * 1024),
                                             (__attribute__((address_space(3))) void*)(sb + j * 1024), 16, 0, 0);
    };

    floatx16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    // fragment addressing: physical row = block*32 + li; chunk position (2*ks + lh) ^ chunk_swizzle(row)
    const int a_row_off = ((wm * FM) * 32 + li) * ROWB;
    const int b_row_off = A_BYTES + ((wn * FN) * 32 + li) * ROWB;
    const int sw = chunk_swizzle(li);

    half8_t af[2][FM], bf[2][FN];
    auto read_frags = [&](const char* base, int ks, int buf) {
        const int ch = (((ks << 1) | lh) ^ sw) << 4;
#pragma unroll
        for (int i = 0; i < FM; i++) af[buf][i] = *reinterpret_cast<const half8_t*>(base + a_row_off + i * 32 * ROWB + ch);
#pragma unroll
        for (int j = 0; j < FN; j++) bf[buf][j] = *reinterpret_cast<const half8_t*>(base + b_row_off + j * 32 * ROWB + ch);
    };
    auto mfma_block = [&](int buf) {
#pragma unroll
        for (int i = 0; i < FM; i++)
#pragma unroll
            for (int j = 0; j < FN; j++)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[buf][i], bf[buf][j], acc[i][j], 0, 0, 0);
    };

    // prologue: fill the ring, wait for tile 0
#pragma unroll
    for (int t = 0; t < NSTAGE; t++) issue_loads(t, t);
    wait_vmcnt<(NSTAGE - 1) * LOADS>();
    __syncthreads();
    read_frags(lds, 0, 0);

    // Steady state, per k tile: the second half's fragments are fetched under the first half's
    // MFMAs; then ONE barrier (next tile landed + everybody is done reading this slot), the
    // next tile's first fragments and the refill of this slot are issued under the second
    // half's MFMAs.
    // Instruction order inside each half is pinned: one LDS read (and, in the second half, one
    // global request) behind each MFMA, so that their issue slots fall into the 32 cycles the
    // matrix pipe spends on the MFMA before and the pipe never waits for the wave to get through a
    // burst of memory instructions.
    constexpr int NMF = FM * FN, NRD = FM + FN;
    for (int kt = 0; kt < nk; kt++) {
        const int slot = kt % NSTAGE;
        const char* base = lds + slot * STAGE;
        read_frags(base, 1, 1);
        mfma_block(0);
#pragma unroll
        for (int i = 0; i < NMF; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                 // MFMA
            if (i < NRD) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);    // LDS read
        }
        __builtin_amdgcn_sched_barrier(0);      // keep the MFMAs above the waits: they hide the read latency
        wait_vmcnt<(NSTAGE - 2) * LOADS>();    // tile kt+1 has landed (this wave's share)
        wait_lgkmcnt0();                        // this wave's reads of slot kt are complete
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        const int nslot = (kt + 1) % NSTAGE;
        read_frags(lds + nslot * STAGE, 0, 0);  // after the last tile: a dummy tile, never multiplied
        issue_loads(kt + NSTAGE, slot);
        mfma_block(1);
#pragma unroll
        for (int i = 0; i < NMF; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (i < NRD) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            else if (i - NRD < LOADS) __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);   // global -> LDS request
        }
    }
    wait_vmcnt<0>();                            // drain the dummy tail requests before LDS goes away

    // ---- epilogue: bias, activation, predicated (vector when legal) store ------------------
    // Bias values are fetched in batches (all of a 32-row block at once, or once per lane when
    // the bias does not vary along rows) so the stores never wait on one load each.
    const float* bias = p.bias ? p.bias + bi * p.bias_sn + bj * p.bias_sc : nullptr;
    const int gn = n0 + wn * TN + li * FN;                // first of this lane's FN columns
    const bool vec_ok = ((p.ldc & 3) == 0) && ((reinterpret_cast<uintptr_t>(C) & 15) == 0) && (gn + FN <= p.N);
    float bcol[FN];
    const bool bias_rowless = bias && p.bias_sm == 0;
#pragma unroll
    for (int j = 0; j < FN; j++) bcol[j] = (bias_rowless && gn + j < p.N) ? bias[(long)(gn + j) * p.bias_sk] : 0.f;
#pragma unroll
    for (int i = 0; i < FM; i++) {
        float bv[16][FN];
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int gm = m0 + wm * TM + ((r >> 2) * 8 + lh * 4 + (r & 3)) * FM + i;
#pragma unroll
            for (int j = 0; j < FN; j++)
                bv[r][j] = (bias && !bias_rowless && gm < p.M && gn + j < p.N)
                               ? bias[(long)gm * p.bias_sm + (long)(gn + j) * p.bias_sk]
                               : bcol[j];
        }
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int im = (r >> 2) * 8 + lh * 4 + (r & 3);
            const int gm = m0 + wm * TM + im * FM + i;
            if (gm >= p.M) continue;
            float v[FN];
#pragma unroll
            for (int j = 0; j < FN; j++) {
                float x = acc[i][j][r] + bv[r][j];
                if (p.relu) x = x > 0.f ? x : 0.f;
                v[j] = x;
            }
            float* dst = C + (long)gm * p.ldc + gn;
            if (vec_ok) {
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

// Same tiles, ring and rasterisation with v_mfma_f32_16x16x32_f16: one MFMA covers the whole 32-wide
// k tile of a 16-row block, a wave's tile is (TM/16) x (TN/16) blocks. A register-only loop of this
// instruction sustains 1.9 PFLOP/s on random fp16 data on an MI355X against 1.62 PFLOP/s for
// 32x32x16 (the chip is power-limited on real data).
// Image rows are interleaved in 16-row blocks (phys_row_of(r, TM/16 or TN/16, 16)): a lane ends
// up with TN/16 = 8 adjacent output columns of 4 rows per A block.
template <int BM, int BN, int WM, int WN, int NSTAGE>
__global__ __launch_bounds__(WM* WN * 64, (BM < CVT_ROWS ? 2 : 1)) void gemm_h16x_kernel(const H16Args p) {
    static_assert((BM == CVT_ROWS || BM * 2 == CVT_ROWS) && BN == CVT_ROWS, "must match the workspace block image");
    constexpr int BK = CVT_K, ROWB = 64;
    constexpr int NW = WM * WN;
    constexpr int TM = BM / WM, TN = BN / WN, FM = TM / 16, FN = TN / 16;
    constexpr int A_BYTES = BM * ROWB, B_BYTES = BN * ROWB, STAGE = A_BYTES + B_BYTES;
    constexpr int A_LOADS = BM / 16 / NW, B_LOADS = BN / 16 / NW;   // wave-wide 1 KiB loads (16 rows) per wave
    constexpr int LOADS = A_LOADS + B_LOADS;
    static_assert(BM % (16 * NW) == 0 && BN % (16 * NW) == 0, "tile/wave mismatch");
    static_assert((NSTAGE - 1) * LOADS < 64, "too many loads in flight for vmcnt");
    static_assert(FN == 8 && FM % 2 == 0, "the epilogue stores 8 adjacent columns per lane");

    extern __shared__ __attribute__((aligned(1024))) char lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int l16 = lane & 15, lq = lane >> 4;

    // one-dimensional grid over (batch member, tile), member-major, one contiguous eighth per XCD
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
    const long a_idx = (long)(p.a_bcast_n ? 0 : bi) * p.a_cn + (p.a_bcast_c ? 0 : bj);
    const long b_idx = (long)(p.b_bcast_n ? 0 : bi) * p.b_cn + (p.b_bcast_c ? 0 : bj);
    const _Float16* __restrict__ A = p.A + a_idx * p.a_batch;
    const _Float16* __restrict__ B = p.B + b_idx * p.b_batch;
    float* __restrict__ C = p.C + bi * p.c_sn + bj * p.c_sc;

    const int nk = p.Kp / BK;
    constexpr int A_BLOCK = CVT_ROWS * ROWB, A_PER_BLOCK = CVT_ROWS / BM;
    const char* a_tile = reinterpret_cast<const char*>(A) + (long)(tile_m / A_PER_BLOCK) * nk * A_BLOCK +
                         (tile_m % A_PER_BLOCK) * A_BYTES + wave * A_LOADS * 1024 + lane * 16;
    const char* b_tile = reinterpret_cast<const char*>(B) + (long)tile_n * nk * B_BYTES + wave * B_LOADS * 1024 + lane * 16;

    // Past the end the last tile is requested again (into a slot nobody reads any more) so that
    // the number of loads in flight, which the vmcnt waits count on, is the same in every step.
    auto issue_loads = [&](int kt, int stage) {
        const int kc = kt < nk ? kt : nk - 1;
        char* sa = lds + stage * STAGE + wave * A_LOADS * 1024;
        char* sb = lds + stage * STAGE + A_BYTES + wave * B_LOADS * 1024;
        const char* ak = a_tile + (long)kc * A_BLOCK;
        const char* bk = b_tile + (long)kc * B_BYTES;
#pragma unroll
        for (int j = 0; j < A_LOADS; j++)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(ak + j * 1024),
                                             (__attribute__((address_space(3))) void*)(sa + j * 1024), 16, 0, 0);
#pragma unroll
        for (int j = 0; j < B_LOADS; j++)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(bk + j * 1024),
                                             (__attribute__((address_space(3))) void*)(sb + j * 1024), 16, 0, 0);
    };

    // Accumulators are named by issue position: on this chip back-to-back MFMAs run fastest when
    // they walk the accumulator registers in ascending order (register-only loop, random fp16 data:
    // 1.92 PFLOP/s in that order, 1.73 with a stride of 8 accumulators, 1.41 with a permuted order;
    // which A / B fragments they take makes no difference). Position t = h*HALF + i*4 + jj is the
    // product of A block i and B block j = 4h + jj: two passes over the A blocks, each against one
    // half of the B blocks, so that every fragment is free again at least 29 MFMAs before its next use
    // and one fragment set is enough.
    constexpr int HALF = FM * 4, NPOS = 2 * HALF;
    // request number q (A pieces first, then B pieces) of k tile kt into ring slot `stage`
    auto issue_load = [&](int kt, int stage, int q) {
        const int kc = kt < nk ? kt : nk - 1;
        const bool is_a = q < A_LOADS;
        const int j = is_a ? q : q - A_LOADS;
        char* dst = lds + stage * STAGE + (is_a ? 0 : A_BYTES) + (wave * (is_a ? A_LOADS : B_LOADS) + j) * 1024;
        const char* src = is_a ? a_tile + (long)kc * A_BLOCK + j * 1024 : b_tile + (long)kc * B_BYTES + j * 1024;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                         (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
    };
    floatx4 acc[NPOS];
#pragma unroll
    for (int t = 0; t < NPOS; t++)
#pragma unroll
        for (int r = 0; r < 4; r++) acc[t][r] = 0.f;

    // fragment addressing: physical row = block*16 + l16, the lane's 8 k values are chunk lq,
    // stored at chunk position lq ^ chunk_swizzle(row)
    const int frag_off = l16 * ROWB + ((lq ^ chunk_swizzle(l16)) << 4);
    const int a_off = (wm * FM) * 16 * ROWB + frag_off;
    const int b_off = A_BYTES + (wn * FN) * 16 * ROWB + frag_off;

    half8_t af[FM], bf[FN];
    auto read_a = [&](const char* base, int i) { af[i] = *reinterpret_cast<const half8_t*>(base + a_off + i * 16 * ROWB); };
    auto read_b = [&](const char* base, int j) { bf[j] = *reinterpret_cast<const half8_t*>(base + b_off + j * 16 * ROWB); };
    auto mfma_at = [&](int t) {
        const int h = t / HALF, i = (t % HALF) / 4, j = 4 * h + (t & 3);
        // Written as assembly so that the accumulator is updated in place in the accumulation
        // registers: given the builtin, the register allocator moves a dozen of the 64 accumulators
        // through a temporary every k tile (four copy instructions per MFMA).
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[t]) : "v"(af[i]), "v"(bf[j]));
    };

    // prologue: fill the ring, wait for tile 0, read its fragments
#pragma unroll
    for (int t = 0; t < NSTAGE; t++) issue_loads(t, t);
    wait_vmcnt<(NSTAGE - 1) * LOADS>();
    __syncthreads();
#pragma unroll
    for (int j = 0; j < FN; j++) read_b(lds, j);
#pragma unroll
    for (int i = 0; i < FM; i++) read_a(lds, i);

    // One k tile: PRE MFMAs, then ONE barrier (tile kt+1 has landed for every wave, and every
    // wave has finished reading slot kt: its last reads were issued at the end of the previous
    // tile), then the refill of slot kt and, as each fragment is used for the last time, the read
    // of its successor from tile kt+1 — one memory instruction behind one MFMA.
    constexpr int PRE = 16 < HALF - 4 ? 16 : HALF - 4 - LOADS;
    static_assert(PRE >= 1 && PRE + LOADS <= HALF - 4, "the refill must be issued before the first fragment is re-read");
    for (int kt = 0; kt < nk; kt++) {
        const char* nxt = lds + ((kt + 1) % NSTAGE) * STAGE;   // after the last tile: a dummy tile, never multiplied
        // a scheduling fence behind every position keeps the instruction order exactly as written
#pragma unroll
        for (int t = 0; t < PRE; t++) {
            mfma_at(t);
            __builtin_amdgcn_sched_barrier(0);
        }
        wait_vmcnt<(NSTAGE - 2) * LOADS>();    // tile kt+1 has landed (this wave's share)
        wait_lgkmcnt0();                        // this wave's reads of slot kt are complete
#ifndef ABL_NOBARRIER
        __syncthreads();
#endif
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = PRE; t < NPOS; t++) {
            mfma_at(t);
#ifndef ABL_NOLOAD
            if (t - PRE < LOADS) issue_load(kt + NSTAGE, kt % NSTAGE, t - PRE);
#endif
#ifndef ABL_NOFRAG
            // last use of B block jj of the first half: position HALF - 4 + jj
            if (t >= HALF - 4 && t < HALF) read_b(nxt, t - (HALF - 4));
            // last use of A block i: position HALF + 4 i + 3
            if (t >= HALF && (t & 3) == 3) read_a(nxt, (t - HALF) / 4);
            // last use of B block 4 + jj: position NPOS - 4 + jj
            if (t >= NPOS - 4) read_b(nxt, 4 + t - (NPOS - 4));
#endif
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    wait_vmcnt<0>();                            // drain the dummy tail requests before LDS goes away
    // the last MFMAs must have left the pipeline before ordinary instructions read their results
    // (the compiler does not know that the assembly statements above are MFMAs)
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

    // ---- epilogue: bias, activation, predicated (vector when legal) store ------------------
    // Accumulator of (A block i, B block j), register r: row (lq*4 + r) of the block, column l16; with the interleaved
    // images that is output row wm*TM + (lq*4 + r)*FM + i and output column wn*TN + l16*FN + j.
    const float* bias = p.bias ? p.bias + bi * p.bias_sn + bj * p.bias_sc : nullptr;
    const int gn = n0 + wn * TN + l16 * FN;               // first of this lane's FN columns
    const bool vec_ok = ((p.ldc & 3) == 0) && ((reinterpret_cast<uintptr_t>(C) & 15) == 0) && (gn + FN <= p.N);
    float bcol[FN];
    const bool bias_rowless = bias && p.bias_sm == 0;
#pragma unroll
    for (int j = 0; j < FN; j++) bcol[j] = (bias_rowless && gn + j < p.N) ? bias[(long)(gn + j) * p.bias_sk] : 0.f;
#pragma unroll
    for (int i = 0; i < FM; i++) {
        float bv[4][FN];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int gm = m0 + wm * TM + (lq * 4 + r) * FM + i;
#pragma unroll
            for (int j = 0; j < FN; j++)
                bv[r][j] = (bias && !bias_rowless && gm < p.M && gn + j < p.N)
                               ? bias[(long)gm * p.bias_sm + (long)(gn + j) * p.bias_sk]
                               : bcol[j];
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int gm = m0 + wm * TM + (lq * 4 + r) * FM + i;
            if (gm >= p.M) continue;
            float v[FN];
#pragma unroll
            for (int j = 0; j < FN; j++) {
                float x = acc[(j >> 2) * HALF + i * 4 + (j & 3)][r] + bv[r][j];
                if (p.relu) x = x > 0.f ? x : 0.f;
                v[j] = x;
            }
            float* dst = C + (long)gm * p.ldc + gn;
            if (vec_ok) {
                floatx4 o0 = {v[0], v[1], v[2], v[3]}, o1 = {v[4], v[5], v[6], v[7]};
                *reinterpret_cast<floatx4*>(dst) = o0;
                *reinterpret_cast<floatx4*>(dst + 4) = o1;
            } else {
#pragma unroll
                for (int j = 0; j < FN; j++)
                    if (gn + j < p.N) dst[j] = v[j];
            }
        }
    }
}

// ---- host side -----------------------------------------------------------------------------
static inline long round_up(long v, long q) { return (v + q - 1) / q * q; }

bool gemm_h16_applicable(const nzhip_gemm_desc& d) {
    // Worth it when each operand element is re-read by many tiles, i.e. when the GEMM does far
    // more work per operand byte than the extra rounding pass moves. Measured on MI355X
    // (microseconds, fused / two-pass): 4096x1024x4096 66 / 60, 3072^3 136 / 102, 4096^3 197 / 163,
    // but 2048^3 44 / 53, 4096x256x4096 30 / 36, 8192x512x8192 160 / 168 (short contractions leave
    // the rounding pass and the C stores nothing to hide behind). Shapes that are not whole
    // 256x256x32 tiles take the fused kernel's predicated instance, which is much slower, so the
    // threshold is lower for them: 2500^3 101 / 68, 5000x1000x5000 156 / 94, 2000^3 56 / 55.
    if (d.M < 512 || d.N < 512 || d.K < 768) return false;
    const double flops = 2.0 * d.M * d.N * d.K;
    const double cvt_bytes = 6.0 * ((double)d.M * d.K + (double)d.N * d.K);
    const bool whole_tiles = d.M % 256 == 0 && d.N % 256 == 0 && d.K % 32 == 0 && d.lda % 4 == 0 && d.ldb % 4 == 0 &&
                             d.ldc % 4 == 0;
    return flops / cvt_bytes >= (whole_tiles ? 512.0 : 300.0);
}

int gemm_h16_dispatch(const nzhip_gemm_desc& d, hipStream_t s, int waves, int mfma) {
    constexpr int BM = 256, BN = 256, BK = 32, NSTAGE = 4;
    const long Mp = round_up(d.M, BM), Np = round_up(d.N, BN), Kp = round_up(d.K, BK);
    const bool a_trans = d.a_layout == NZHIP_LAYOUT_TRANS, b_trans = d.b_layout == NZHIP_LAYOUT_TRANS;
    // workspace holds one rounded copy per DISTINCT batch member of each operand
    const long a_n = d.a_stride_n ? d.batch_n : 1, a_c = d.a_stride_c ? d.batch_c : 1;
    const long b_n = d.b_stride_n ? d.batch_n : 1, b_c = d.b_stride_c ? d.batch_c : 1;
    const size_t a_elems = (size_t)Mp * Kp, b_elems = (size_t)Np * Kp;
    const size_t a_total = a_elems * a_n * a_c, b_total = b_elems * b_n * b_c;
    _Float16* ws = nullptr;
    if (int rc = workspace_alloc(reinterpret_cast<void**>(&ws), (a_total + b_total) * sizeof(_Float16), s)) return rc;
    _Float16* Ah = ws;
    _Float16* Bh = ws + a_total;

    const int nkt = (int)(Kp / BK);
    auto operand = [&](_Float16* dst, const float* src, long R, long ld, long sc, size_t elems, int fr) {
        CvtOperand o;
        o.dst = dst;
        o.src = src;
        o.R = (int)R;
        o.ld = ld;
        o.src_batch = sc;
        o.dst_batch = (long)elems;
        o.vec = ((ld & 3) == 0) && ((reinterpret_cast<uintptr_t>(src) & 15) == 0) && ((sc & 3) == 0);
        o.fr = fr;
        return o;
    };
    auto convert = [&](_Float16* dst, const float* src, long R, long Rp, bool k_contig, long ld, long nb, long cb,
                       long sn, long sc, size_t elems, int fr, int blk) -> int {
        for (long i = 0; i < nb; i++) {
            // the c axis of one n is a plain strided batch -> one launch per n
            const CvtOperand o = operand(dst + (size_t)i * cb * elems, src + i * sn, R, ld, sc, elems, fr);
            dim3 grid((unsigned)nkt, (unsigned)(Rp / CVT_ROWS), (unsigned)cb);
            if (k_contig)
                hipLaunchKernelGGL(cvt_block_kernel<true>, grid, dim3(256), 0, s, o, (int)d.K, nkt, blk);
            else
                hipLaunchKernelGGL(cvt_block_kernel<false>, grid, dim3(256), 0, s, o, (int)d.K, nkt, blk);
        }
        hipError_t e = hipGetLastError();
        return e == hipSuccess ? NZHIP_OK : set_hip_error(e, "fp16 rounding pass launch");
    };
    // both operands in one launch when they have the same batch structure (one n, equal c extents)
    auto convert_pair = [&](int fr_a, int fr_b, int blk) -> int {
        const CvtOperand oa = operand(Ah, d.A, d.M, d.lda, d.a_stride_c, a_elems, fr_a);
        const CvtOperand ob = operand(Bh, d.B, d.N, d.ldb, d.b_stride_c, b_elems, fr_b);
        const int a_blocks = (int)(Mp / CVT_ROWS), b_blocks = (int)(Np / CVT_ROWS);
        dim3 grid((unsigned)nkt, (unsigned)(a_blocks + b_blocks), (unsigned)a_c);
        const bool ka = !a_trans, kb = b_trans;
        if (ka && kb) hipLaunchKernelGGL((cvt_pair_kernel<true, true>), grid, dim3(256), 0, s, oa, ob, a_blocks, (int)d.K, nkt, blk);
        else if (ka) hipLaunchKernelGGL((cvt_pair_kernel<true, false>), grid, dim3(256), 0, s, oa, ob, a_blocks, (int)d.K, nkt, blk);
        else if (kb) hipLaunchKernelGGL((cvt_pair_kernel<false, true>), grid, dim3(256), 0, s, oa, ob, a_blocks, (int)d.K, nkt, blk);
        else hipLaunchKernelGGL((cvt_pair_kernel<false, false>), grid, dim3(256), 0, s, oa, ob, a_blocks, (int)d.K, nkt, blk);
        hipError_t e = hipGetLastError();
        return e == hipSuccess ? NZHIP_OK : set_hip_error(e, "fp16 rounding pass launch");
    };
    // Kernel variants (waves: 0 = choose, 4 / 8 / 2 = force):
    //   8: 256 x 256 tile, 4 x 2 waves (two per SIMD, 128 accumulators each): the memory instructions of one
    //      wave issue under the MFMAs of the other (8192^3 with 16x16x32: 1.08 ms against 1.10 ms with 4 waves)
    //   4: 256 x 256 tile, 2 x 2 waves (one wave per SIMD, 256 accumulators), 4-stage ring, 1 workgroup per CU
    //   2: 128 x 256 tile, 2 x 2 waves, 3-stage ring of 72 KiB: two workgroups share a CU, so the output
    //      stores and ring fill of one overlap the MFMAs of the other -- for products with few tiles
    // mfma: 0 = choose (16), 16 = v_mfma_f32_16x16x32_f16, 32 = v_mfma_f32_32x32x16_f16 (8192^3: 1.10 / 1.13 ms
    // with 4 waves; the 32x32x16 loop is kept for comparison).
    static const char* waves_env = getenv("NZHIP_H16_WAVES");
    if (waves == 0 && waves_env) waves = atoi(waves_env);
    static const char* mfma_env = getenv("NZHIP_H16_MFMA");             // 16 | 32: benchmarking only
    if (mfma == 0 && mfma_env) mfma = atoi(mfma_env);
    const bool mf16 = mfma != 32;
    if (waves != 2 && waves != 4 && waves != 8) {
        const long t256 = (Mp / 256) * (Np / 256) * d.batch_n * d.batch_c;
        waves = t256 < 2 * device_cu_count() ? 2 : (mf16 ? 8 : 4);
    }
    const bool half_m = waves == 2;
    const int wm_waves = waves == 8 ? 4 : 2;
    const int blk = mf16 ? 16 : 32;                                     // rows per MFMA block
    const int fr_a = (half_m ? 64 : 256 / wm_waves) / blk, fr_b = 128 / blk;   // blocks per wave tile
    int rc;
    if (a_n == 1 && b_n == 1 && a_c == b_c && (Mp + Np) / CVT_ROWS <= 65535) {
        rc = convert_pair(fr_a, fr_b, blk);
    } else {
        rc = convert(Ah, d.A, d.M, Mp, !a_trans, d.lda, a_n, a_c, d.a_stride_n, d.a_stride_c, a_elems, fr_a, blk);
        if (rc == NZHIP_OK)
            rc = convert(Bh, d.B, d.N, Np, b_trans, d.ldb, b_n, b_c, d.b_stride_n, d.b_stride_c, b_elems, fr_b, blk);
    }
    if (rc == NZHIP_OK) {
        H16Args a;
        a.A = Ah;
        a.B = Bh;
        a.C = d.C;
        a.bias = d.bias;
        a.M = (int)d.M;
        a.N = (int)d.N;
        a.Kp = (int)Kp;
        a.ldc = d.ldc;
        a.batch_c = (int)d.batch_c;
        a.batch = (int)(d.batch_n * d.batch_c);
        a.a_batch = (long)a_elems;
        a.b_batch = (long)b_elems;
        a.a_bcast_n = d.a_stride_n == 0;
        a.a_bcast_c = d.a_stride_c == 0;
        a.b_bcast_n = d.b_stride_n == 0;
        a.b_bcast_c = d.b_stride_c == 0;
        a.a_cn = (int)a_c;
        a.b_cn = (int)b_c;
        a.c_sn = d.c_stride_n;
        a.c_sc = d.c_stride_c;
        a.bias_sn = d.bias_stride_n;
        a.bias_sc = d.bias_stride_c;
        a.bias_sm = d.bias_stride_row;
        a.bias_sk = d.bias_stride_col;
        a.relu = d.activation == NZHIP_ACT_RELU;
        a.tiles_m = (int)(Mp / (half_m ? 128 : BM));
        a.tiles_n = (int)(Np / BN);
        a.group_m = half_m ? 8 : 4;
        const size_t lds_bytes = half_m ? (size_t)3 * (128 + BN) * 64 : (size_t)NSTAGE * (BM + BN) * 64;
        void (*kfn)(const H16Args) = half_m          ? gemm_h16_kernel<128, BN, 2, 2, 3>
                                     : wm_waves == 4 ? gemm_h16_kernel<BM, BN, 4, 2, NSTAGE>
                                                     : gemm_h16_kernel<BM, BN, 2, 2, NSTAGE>;
        if (mf16)
            kfn = half_m          ? gemm_h16x_kernel<128, BN, 2, 2, 3>
                  : wm_waves == 4 ? gemm_h16x_kernel<BM, BN, 4, 2, NSTAGE>
                                  : gemm_h16x_kernel<BM, BN, 2, 2, NSTAGE>;
        if (rc == NZHIP_OK)
            rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kfn), (int)lds_bytes, "hipFuncSetAttribute(gemm_h16)");
        if (rc == NZHIP_OK) {
            dim3 grid((unsigned)((int64_t)a.tiles_m * a.tiles_n * a.batch));
            hipLaunchKernelGGL(kfn, grid, dim3(wm_waves * 2 * 64), lds_bytes, s, a);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) rc = set_hip_error(e, "gemm_h16 kernel launch");
        }
    }
    int rc2 = workspace_free(ws, s);
    return rc ? rc : rc2;
}

}  // namespace nzhip
