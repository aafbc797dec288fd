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

#include <atomic>
#include <mutex>

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
// the inverse: logical tile row held at physical row pr
__device__ __forceinline__ int logical_row_of(int pr, int fr, int blk) {
    const int b = pr / blk, in = pr % blk;
    return (b / fr) * (blk * fr) + in * fr + (b % fr);
}

// K_CONTIG: source element (r, k) at src[r*ld + k]; otherwise at src[k*ld + r].
struct CvtOperand {
    _Float16* dst;
    const float* src;
    int R;                      // rows of the operand (output rows for A, output columns for B)
    long ld, src_batch, dst_batch;
    int vec, fr;
};

// WHOLE: the block lies inside the operand and 16-byte loads are legal, so the eight requests of a thread carry no
// condition and are all in flight before the first is used (a launch of few blocks is bound by that latency).
template <bool K_CONTIG, bool WHOLE = false>
__device__ __forceinline__ void cvt_block(char* img, const CvtOperand& o, int K, int nkt, int blk, int kt, int rb, int member) {
    _Float16* dst = o.dst;
    const int R = o.R, vec = o.vec, fr = o.fr;
    const long ld = o.ld, dst_batch = o.dst_batch;
    const float* s = o.src + (long)member * o.src_batch;
    const int t = threadIdx.x;
    const int r0 = rb * CVT_ROWS, k0 = kt * CVT_K;
    if (K_CONTIG) {
        // 8 threads per row (one float4 each), 32 rows per pass. The threads walk the PHYSICAL rows of the
        // image, so a wave's 8-byte stores cover 512 contiguous bytes of LDS (conflict-free); walking the
        // logical rows puts rows 16 apart (1 KiB, the same banks) into one store instruction. In global
        // memory a row's 32 values are one 128-byte line either way.
        const int k4 = t & 7, rr = t >> 3;
        floatx4 whole[8];
        if (WHOLE) {
#pragma unroll
            for (int pass = 0; pass < 8; pass++)
                whole[pass] = *reinterpret_cast<const floatx4*>(s + (long)(r0 + logical_row_of(rr + pass * 32, fr, blk)) * ld + k0 + k4 * 4);
        }
#pragma unroll
        for (int pass = 0; pass < 8; pass++) {
            const int pr_ = rr + pass * 32, lr = logical_row_of(pr_, fr, blk), r = r0 + lr, k = k0 + k4 * 4;
            floatx4 v = {0.f, 0.f, 0.f, 0.f};
            const float* q = s + (long)r * ld + k;
            if (WHOLE) {
                v = whole[pass];
            } else if (r < R) {
                if (vec && k + 4 <= K) {
                    v = *reinterpret_cast<const floatx4*>(q);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (k + e < K) v[e] = q[e];
                }
            }
            half4_t h = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
            const int pr = pr_;
            const int pos = (k4 >> 1) ^ chunk_swizzle(pr);
            *reinterpret_cast<half4_t*>(img + pr * 64 + pos * 16 + (k4 & 1) * 8) = h;
        }
    } else {
        // 64 threads per k row (one float4 of 4 rows each), 4 k rows per pass
        const int r4 = t & 63, kk0 = t >> 6;
        floatx4 whole[8];
        if (WHOLE) {
#pragma unroll
            for (int pass = 0; pass < 8; pass++)
                whole[pass] = *reinterpret_cast<const floatx4*>(s + (long)(k0 + kk0 + pass * 4) * ld + r0 + r4 * 4);
        }
#pragma unroll
        for (int pass = 0; pass < 8; pass++) {
            const int kk = kk0 + pass * 4, k = k0 + kk, lr = r4 * 4, r = r0 + lr;
            floatx4 v = {0.f, 0.f, 0.f, 0.f};
            const float* q = s + (long)k * ld + r;
            if (WHOLE) {
                v = whole[pass];
            } else if (k < K) {
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
            if (gm >= p.M) continue;
            float v[FN];
#pragma unroll
            for (int j = 0; j < FN; j++) {
                float x = acc[i][j][r] + (bias_rows ? bvs[(i * 2 + (r >> 3)) & 1][r & 7][j] : bcol[j]);
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
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = PRE; t < NPOS; t++) {
            mfma_at(t);
            if (t - PRE < LOADS) issue_load(kt + NSTAGE, kt % NSTAGE, t - PRE);
            // last use of B block jj of the first half: position HALF - 4 + jj
            if (t >= HALF - 4 && t < HALF) read_b(nxt, t - (HALF - 4));
            // last use of A block i: position HALF + 4 i + 3
            if (t >= HALF && (t & 3) == 3) read_a(nxt, (t - HALF) / 4);
            // last use of B block 4 + jj: position NPOS - 4 + jj
            if (t >= NPOS - 4) read_b(nxt, 4 + t - (NPOS - 4));
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
    // A bias that varies along rows (a bias matrix, C itself when a gradient is accumulated in place) is requested one
    // block of rows ahead of the stores that need it: a load issued after stores is not counted as returned before
    // those stores are acknowledged, so requesting block i after storing block i - 1 made every block wait for the
    // one before. 16-byte loads when the bias rows are contiguous and aligned like the rows of C.
    const bool bias_rows = bias && !bias_rowless;
    const bool bias_vec = bias_rows && p.bias_sk == 1 && (p.bias_sm & 3) == 0 && (reinterpret_cast<uintptr_t>(bias) & 15) == 0 &&
                          gn + FN <= p.N;
    float bvs[2][4][FN];
    auto bias_request = [&](float (&bv)[4][FN], const int i) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int gm = m0 + wm * TM + (lq * 4 + r) * FM + i;
            const float* bp = bias + (long)(gm < p.M ? gm : 0) * p.bias_sm;
            if (bias_vec) {
#pragma unroll
                for (int q = 0; q < FN / 4; q++) {
                    const floatx4 v = *reinterpret_cast<const floatx4*>(bp + gn + 4 * q);
#pragma unroll
                    for (int e = 0; e < 4; e++) bv[r][4 * q + e] = v[e];
                }
            } else {
#pragma unroll
                for (int j = 0; j < FN; j++) bv[r][j] = bp[gn + j < p.N ? (long)(gn + j) * p.bias_sk : 0];
            }
        }
    };
    if (bias_rows) bias_request(bvs[0], 0);
#pragma unroll
    for (int i = 0; i < FM; i++) {
        if (bias_rows && i + 1 < FM) bias_request(bvs[(i + 1) & 1], i + 1);
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int gm = m0 + wm * TM + (lq * 4 + r) * FM + i;
            if (gm >= p.M) continue;
            float v[FN];
#pragma unroll
            for (int j = 0; j < FN; j++) {
                float x = acc[(j >> 2) * HALF + i * 4 + (j & 3)][r] + (bias_rows ? bvs[i & 1][r][j] : bcol[j]);
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

// ---- both passes in one kernel for very large products --------------------------------------------
// The rounding pass is memory-bound and the MFMA pass leaves most of the HBM bandwidth idle, so for
// products with many tiles the two are overlapped: the workgroups of the GEMM round, inside their k
// loops, the operand blocks that will be needed NEXT, and counters in memory tell a workgroup when
// the blocks it is about to request have been written by everybody.
//
// Schedule. The grid is cut into waves of 256 workgroups (one per CU); wave w computes the 16 x 16
// tile block (sbm, sbn) of C, the blocks taken in boustrophedon order so that consecutive waves
// share the A rows or the B columns. A k loop is cut into panels of COOP_KP k tiles. Stage (w, p) is
// the set of fp16 image blocks that wave w needs in panel p and that no earlier wave needed (the A
// blocks of a tile-block row when it is entered, the B blocks only in the first tile-block row).
// Stage (0, 0) is rounded by coop_prologue_kernel; every other stage is rounded by the 256
// workgroups of the wave that runs just before it is needed: stage (w, p + 1) during panel p of
// wave w, stage (w + 1, 0) during the last panel of wave w. A stage has at most 32 x COOP_KP blocks,
// i.e. at most 4 per workgroup, 16 fp32 values per thread and block.
//
// A block goes global fp32 -> registers -> fp16 in a 16 KiB LDS staging area (the same image layout
// as cvt_block writes) -> linear 16-byte stores, spread over four k tiles. The stores carry the sc1
// bit (device scope: they are written through the L2 of the writing XCD, which the other XCDs do
// not snoop); once a wave's stores have completed (vmcnt 0) and the workgroup has met at the k
// loop's barrier, one lane adds 1 to the stage's counter with a device-scope atomic. A consumer reads
// the counter with a device-scope load a few k tiles before it needs the stage and, in the normal
// case, finds 256 there; otherwise it sleeps and polls, at most spin_limit times (then it counts a
// time-out in g_coop_timeouts and goes on, so every wave always reaches the end of the kernel). No
// cache invalidation is needed on the consumer side: a block's lines cannot be in a cache before
// they are first requested, they are first requested after the counter has been seen complete, and
// all caches are invalidated at kernel boundaries.
// Completion of stage (w, 0) implies completion of every earlier stage (its producers have passed
// the checks of all stages before it), so the one check a workgroup makes before its first request
// covers the operand blocks that earlier waves rounded.
// Progress: a workgroup only waits for workgroups with a smaller wave number or of its own wave, and
// workgroups are dispatched in order, so with one workgroup per CU and at least 256 CUs nobody waits
// for a workgroup that cannot start.
#ifndef NZHIP_COOP_KP
#define NZHIP_COOP_KP 32
#endif
constexpr int COOP_KP = NZHIP_COOP_KP, COOP_SB = 16, COOP_WG = COOP_SB * COOP_SB;
constexpr int COOP_RND = COOP_KP / 2;           // k tiles of a panel in which rounding work is scheduled (a block every four)

struct CoopArgs {
    H16Args g;
    const float* srcA;
    const float* srcB;
    long lda, ldb;
    unsigned* flags;            // one arrival counter per stage, then the launch's own count of waits that ran out;
                                // zeroed by coop_prologue_kernel
    int sn;                     // tile blocks along N
    int waves, panels;
    unsigned spin_limit;
    int mute;                   // test hook: producers keep their arrivals to themselves, so every wait runs out
};

__device__ unsigned g_coop_timeouts;   // polls that gave up (0 unless the device is shared or smaller than assumed)

template <bool A_KC, bool B_KC>
__global__ __launch_bounds__(256) void coop_prologue_kernel(CvtOperand a, CvtOperand b, int a_blocks, int K, int nkt,
                                                            unsigned* flags, int n_flags) {
    __shared__ __attribute__((aligned(16))) char img[CVT_BLOCK_BYTES];
    if (blockIdx.x == 0 && blockIdx.y == 0)
        for (int i = threadIdx.x; i < n_flags; i += 256) flags[i] = 0;
    const int rb = blockIdx.y;
    if (rb < a_blocks)
        cvt_block<A_KC, true>(img, a, K, nkt, 16, blockIdx.x, rb, 0);
    else
        cvt_block<B_KC, true>(img, b, K, nkt, 16, blockIdx.x, rb - a_blocks, 0);
}

// phys_row_of for 16-row blocks and fr = 1 << lg blocks per wave tile
__device__ __forceinline__ int phys_row16(int r, int lg) {
    const int w = r >> (4 + lg), l = r & ((16 << lg) - 1);
    return (((w << lg) + (l & ((1 << lg) - 1))) << 4) + (l >> lg);
}

template <bool A_KC, bool B_KC>
__global__ __launch_bounds__(512, 1) void gemm_h16c_kernel(const CoopArgs q) {
    constexpr int BM = 256, BN = 256, WN = 2, NSTAGE = 4, ROWB = 64;
    constexpr int TM = 64, TN = 128, FM = TM / 16, FN = TN / 16;
    constexpr int A_BYTES = BM * ROWB, B_BYTES = BN * ROWB, STAGE = A_BYTES + B_BYTES;
    constexpr int A_LOADS = 2, B_LOADS = 2, LOADS = A_LOADS + B_LOADS;
    constexpr int RING = NSTAGE * STAGE;
    const H16Args& p = q.g;

    extern __shared__ __attribute__((aligned(1024))) char lds[];
    char* const stg = lds + RING;                              // 32 KiB staging area of the rounding work

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int l16 = lane & 15, lq = lane >> 4;

    // wave of workgroups, slot in it, tile
    const int wv = blockIdx.x / COOP_WG, slot = blockIdx.x % COOP_WG;
    auto block_of = [&](int w, int& sbm, int& sbn, bool& new_a, bool& new_b) {
        sbm = w / q.sn;
        const int j = w - sbm * q.sn;
        sbn = (sbm & 1) ? q.sn - 1 - j : j;
        new_a = j == 0;
        new_b = sbm == 0;
    };
    int sbm, sbn;
    bool unused_a, unused_b;
    block_of(wv, sbm, sbn, unused_a, unused_b);
    const int xcd = slot & 7, sq = slot >> 3;                  // workgroups go to the XCDs round-robin: 4 x 8 tiles per XCD
    const int tile_m = sbm * COOP_SB + (xcd & 3) * 4 + (sq & 3);
    const int tile_n = sbn * COOP_SB + (xcd >> 2) * 8 + (sq >> 2);
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    const _Float16* __restrict__ A = p.A;
    const _Float16* __restrict__ B = p.B;
    float* __restrict__ C = p.C;
    const int nk = p.Kp / CVT_K;
    const char* a_tile = reinterpret_cast<const char*>(A) + (long)tile_m * nk * A_BYTES + wave * A_LOADS * 1024 + lane * 16;
    const char* b_tile = reinterpret_cast<const char*>(B) + (long)tile_n * nk * B_BYTES + wave * B_LOADS * 1024 + lane * 16;

    auto issue_load = [&](int kt, int stage, int r) {
        const int kc = kt < nk ? kt : nk - 1;
        const bool is_a = r < A_LOADS;
        const int j = is_a ? r : r - A_LOADS;
        char* dst = lds + stage * STAGE + (is_a ? 0 : A_BYTES) + (wave * (is_a ? A_LOADS : B_LOADS) + j) * 1024;
        const char* src = is_a ? a_tile + (long)kc * A_BYTES + j * 1024 : b_tile + (long)kc * B_BYTES + j * 1024;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                         (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
    };

    constexpr int HALF = FM * 4, NPOS = 2 * HALF;
    floatx4 acc[NPOS];
#pragma unroll
    for (int t = 0; t < NPOS; t++)
#pragma unroll
        for (int r = 0; r < 4; r++) acc[t][r] = 0.f;

    const int frag_off = l16 * ROWB + ((lq ^ chunk_swizzle(l16)) << 4);
    const int a_off = (wm * FM) * 16 * ROWB + frag_off;
    const int b_off = A_BYTES + (wn * FN) * 16 * ROWB + frag_off;
    half8_t af[FM], bf[FN];
    auto read_a = [&](const char* base, int i) { af[i] = *reinterpret_cast<const half8_t*>(base + a_off + i * 16 * ROWB); };
    auto read_b = [&](const char* base, int j) { bf[j] = *reinterpret_cast<const half8_t*>(base + b_off + j * 16 * ROWB); };
    auto mfma_at = [&](int t) {
        const int h = t / HALF, i = (t % HALF) / 4, j = 4 * h + (t & 3);
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[t]) : "v"(af[i]), "v"(bf[j]));
    };

    // ---- stage counters -------------------------------------------------------------------------
    auto flag_of = [&](int w, int pn) { return q.flags + (long)w * q.panels + pn; };
    unsigned* const launch_timeouts = q.flags + (long)q.waves * q.panels;
    auto wait_stage = [&](unsigned seen, unsigned* flag) {      // wave 0 only; seen: an earlier reading of *flag
        unsigned v = __builtin_amdgcn_readfirstlane(seen);
        unsigned polls = 0;
        while (v < (unsigned)COOP_WG) {
            __builtin_amdgcn_s_sleep(16);
            v = __builtin_amdgcn_readfirstlane(__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
            if (++polls > q.spin_limit) {
                // Give up, but leave a mark that nobody can miss: the launch's own count (read by every workgroup
                // in front of its result stores, which then write NaN) and the process-wide one (read by the host).
                // The returning atomic is waited for, so the mark is in memory before this workgroup signals
                // anything else.
                if (lane == 0) {
                    atomicAdd(&g_coop_timeouts, 1u);
                    unsigned was = __hip_atomic_fetch_add(launch_timeouts, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    asm volatile("s_waitcnt vmcnt(0)" ::"v"(was) : "memory");
                }
                break;
            }
        }
    };

    // ---- rounding work of this workgroup --------------------------------------------------------
    // Per panel up to four blocks, one every four k tiles. k tile it, it & 3 == 0: the block's 32 KiB of
    // fp32 are requested straight into the staging area (global_load_lds, four 1 KiB pieces per wave: rows
    // of 32 k values when k is contiguous in the source, k rows of 256 values otherwise); the requests sit
    // in front of that k tile's ring requests; requests complete in order, so the ring's own wait three k
    // tiles later (at most 8 requests outstanding) covers them, and the two waits in between allow 12.
    // it & 3 == 3: every thread reads the 8 values of one 16-byte piece of the image from the staging area,
    // rounds them and stores the piece, twice; thread t takes pieces t and 512 + t of the block, so a wave
    // writes 1 KiB runs.
    char* cv_dst = nullptr;                                   // image block in hand (uniform), null = none
    const char* cv_src = nullptr;                             // this lane's first 16 source bytes of it
    long cv_step = 0;                                         // bytes between the wave's four pieces
    int cv_kc = 0, cv_lg = 2;                                 // k contiguous in the source; log2(blocks per wave tile)
    int t_w = 0, t_p = 0, t_na = 0, t_nb = 0, t_sbm = 0, t_sbn = 0;   // the stage being produced in this panel
    bool t_any = false;
    auto begin_panel = [&](int pn) {                          // which stage do we produce during panel pn?
        t_any = false;
        if (pn + 1 < q.panels) { t_w = wv; t_p = pn + 1; t_any = true; }
        else if (wv + 1 < q.waves) { t_w = wv + 1; t_p = 0; t_any = true; }
        if (t_any) {
            bool na, nb;
            block_of(t_w, t_sbm, t_sbn, na, nb);
            t_na = na ? COOP_SB : 0;
            t_nb = nb ? COOP_SB : 0;
        }
    };
    auto begin_block = [&](int n) {                            // n-th block of this workgroup in the stage (uniform)
        const int i = slot + COOP_WG * n;
        cv_dst = nullptr;
        if (!t_any || i >= (t_na + t_nb) * COOP_KP) return;
        const int r = i / COOP_KP, kt = t_p * COOP_KP + i % COOP_KP;
        const bool is_a = r < t_na;
        auto setup = [&](const float* S, const long ld, const _Float16* img, const int rb, const bool kc, const int lg) {
            cv_kc = kc;
            cv_lg = lg;
            const long r0 = (long)rb * CVT_ROWS, k0 = (long)kt * CVT_K;
            if (kc) {       // piece j of wave v: rows 32 v + 8 j .. + 8, lane l -> row + l / 8, k + 4 (l & 7)
                cv_src = reinterpret_cast<const char*>(S + (r0 + wave * 32 + (lane >> 3)) * ld + k0 + 4 * (lane & 7));
                cv_step = 8 * ld * 4;
            } else {        // piece j of wave v: k row 4 v + j, lane l -> 4 rows from 4 l
                cv_src = reinterpret_cast<const char*>(S + (k0 + wave * 4) * ld + r0 + 4 * lane);
                cv_step = ld * 4;
            }
            cv_dst = const_cast<char*>(reinterpret_cast<const char*>(img)) + ((long)rb * nk + kt) * CVT_BLOCK_BYTES;
        };
        // FM = 4 and FN = 8 blocks of 16 rows per wave tile: the images interleave their rows accordingly
        if (is_a) setup(q.srcA, q.lda, A, t_sbm * COOP_SB + r, A_KC, 2);
        else setup(q.srcB, q.ldb, B, t_sbn * COOP_SB + (r - t_na), B_KC, 3);
    };
    auto cv_request = [&]() {                                  // 4 KiB per wave: staging bytes [4096 v, 4096 v + 4096)
#pragma unroll
        for (int j = 0; j < 4; j++)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(cv_src + j * cv_step),
                                             (__attribute__((address_space(3))) void*)(stg + wave * 4096 + j * 1024), 16, 0, 2);   // aux 2 = nt: streamed once, keep it from displacing the tiles in L2
    };
    auto cv_round = [&](int j) {                               // image piece 512 j + t: staging -> registers -> memory
        const int c = j * 512 + tid, pr = c >> 2;
        const int chunk = (c & 3) ^ chunk_swizzle(pr);         // logical 8-wide k chunk held at this position
        // logical row of physical row pr (inverse of phys_row16)
        const int blk16 = pr >> 4, in_blk = pr & 15;
        const int lr = ((blk16 >> cv_lg) << (4 + cv_lg)) + (in_blk << cv_lg) + (blk16 & ((1 << cv_lg) - 1));
        float x[8];
        if (cv_kc) {
            const floatx4 lo = *reinterpret_cast<const floatx4*>(stg + lr * 128 + chunk * 32);
            const floatx4 hi = *reinterpret_cast<const floatx4*>(stg + lr * 128 + chunk * 32 + 16);
#pragma unroll
            for (int e = 0; e < 4; e++) { x[e] = lo[e]; x[4 + e] = hi[e]; }
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++) x[e] = *reinterpret_cast<const float*>(stg + (chunk * 8 + e) * 1024 + lr * 4);
        }
        half8_t h;
#pragma unroll
        for (int e = 0; e < 8; e++) h[e] = (_Float16)x[e];
        // device-scope store (sc1): written through the L2 of this XCD. The no-op keeps the data registers
        // untouched for the cycles in which the store still reads them.
        asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(cv_dst + c * 16), "v"(h) : "memory");
    };

    // ---- prologue ---------------------------------------------------------------------------------
    if (wv > 0 && wave == 0)
        wait_stage(__hip_atomic_load(flag_of(wv, 0), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), flag_of(wv, 0));
    __syncthreads();
#pragma unroll
    for (int t = 0; t < NSTAGE; t++)
#pragma unroll
        for (int r = 0; r < LOADS; r++) issue_load(t, t, r);
    wait_vmcnt<(NSTAGE - 1) * LOADS>();
    __syncthreads();
#pragma unroll
    for (int j = 0; j < FN; j++) read_b(lds, j);
#pragma unroll
    for (int i = 0; i < FM; i++) read_a(lds, i);

    // ---- k loop -----------------------------------------------------------------------------------
    // it: k tile within the panel. DRAIN_IT: every wave waits for its stores, then (behind the barrier)
    // one lane signals; POLL_IT: wave 0 reads the counter of the next panel's stage; CHECK_IT: the k
    // tile in which the first requests of the next panel are issued.
    constexpr int PRE = HALF - 4 - LOADS;
    constexpr int DRAIN_IT = COOP_RND + 2, POLL_IT = COOP_KP - 7, CHECK_IT = COOP_KP - NSTAGE;
    static_assert(DRAIN_IT > COOP_RND && DRAIN_IT < POLL_IT && POLL_IT + 2 < CHECK_IT, "schedule");
    unsigned polled = 0;
    auto k_tile = [&](const int kt, const int slot_c, const int ph) {   // slot_c = kt % NSTAGE, ph = kt & 3 (compile time)
        const int it = kt & (COOP_KP - 1), pn = kt / COOP_KP;
        const char* nxt = lds + ((slot_c + 1) % NSTAGE) * STAGE;
#pragma unroll
        for (int t = 0; t < PRE; t++) {
            mfma_at(t);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (it == DRAIN_IT) wait_vmcnt<0>();                  // this wave's image stores are in memory
        else if ((ph == 1 || ph == 2) && it < COOP_RND && cv_dst) wait_vmcnt<(NSTAGE - 2) * LOADS + 4>();   // + the staging requests of this block
        else wait_vmcnt<(NSTAGE - 2) * LOADS>();              // tile kt+1 has landed (this wave's share)
        wait_lgkmcnt0();
        if (it == CHECK_IT && pn + 1 < q.panels && wave == 0) wait_stage(polled, flag_of(wv, pn + 1));
        // A bare barrier: the waits above name exactly what has to be complete. __syncthreads() would add a
        // workgroup fence, which here (ordinary global loads and stores are in flight) drains every request.
        asm volatile("s_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        if (it == DRAIN_IT && t_any && tid == 0 && !q.mute)
            __hip_atomic_fetch_add(flag_of(t_w, t_p), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (it == POLL_IT && pn + 1 < q.panels && wave == 0)
            polled = __hip_atomic_load(flag_of(wv, pn + 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (ph == 0 && it < COOP_RND) {                             // in front of this k tile's ring requests
            if (it == 0) begin_panel(pn);
            begin_block(it >> 2);
            if (cv_dst) cv_request();
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int t = PRE; t < NPOS; t++) {
            mfma_at(t);
            if (t - PRE < LOADS) issue_load(kt + NSTAGE, slot_c, t - PRE);
            if (t >= HALF - 4 && t < HALF) read_b(nxt, t - (HALF - 4));
            if (t >= HALF && (t & 3) == 3) read_a(nxt, (t - HALF) / 4);
            if (t >= NPOS - 4) read_b(nxt, 4 + t - (NPOS - 4));
            __builtin_amdgcn_sched_barrier(0);
            if ((t == PRE + LOADS || t == HALF + 5) && ph == 3 && it < COOP_RND && cv_dst) {
                cv_round(t == PRE + LOADS ? 0 : 1);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    for (int kt = 0; kt < nk; kt += 4) {
        k_tile(kt, 0, 0);
        k_tile(kt + 1, 1, 1);
        k_tile(kt + 2, 2, 2);
        k_tile(kt + 3, 3, 3);
    }
    wait_vmcnt<0>();
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

    // ---- epilogue (whole tiles only: M and N are multiples of the tile) -----------------------------
    // A wait that ran out anywhere in this launch before this point may have let somebody multiply image blocks
    // that were not complete (this workgroup, or one whose arrival others relied on): the tile is then written
    // as NaN, so that the product cannot be mistaken for a result.
    const bool poisoned =
        __builtin_amdgcn_readfirstlane(__hip_atomic_load(launch_timeouts, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) != 0;
    const float* bias = p.bias;
    const int gn = n0 + wn * TN + l16 * FN;
    float bcol[FN];
    const bool bias_rowless = bias && p.bias_sm == 0;
#pragma unroll
    for (int j = 0; j < FN; j++) bcol[j] = bias_rowless ? bias[(long)(gn + j) * p.bias_sk] : 0.f;
    // a bias that varies along rows is requested one block of rows ahead of the stores that need it (a load issued
    // after stores is not counted as returned before they are acknowledged)
    const bool bias_rows = bias && !bias_rowless;
    const bool bias_vec = bias_rows && p.bias_sk == 1 && (p.bias_sm & 3) == 0 && (reinterpret_cast<uintptr_t>(bias) & 15) == 0;
    float bvs[2][4][FN];
    auto bias_request = [&](float (&bv)[4][FN], const int i) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int gm = m0 + wm * TM + (lq * 4 + r) * FM + i;
            const float* bp = bias + (long)gm * p.bias_sm;
            if (bias_vec) {
#pragma unroll
                for (int q = 0; q < FN / 4; q++) {
                    const floatx4 v = *reinterpret_cast<const floatx4*>(bp + gn + 4 * q);
#pragma unroll
                    for (int e = 0; e < 4; e++) bv[r][4 * q + e] = v[e];
                }
            } else {
#pragma unroll
                for (int j = 0; j < FN; j++) bv[r][j] = bp[(long)(gn + j) * p.bias_sk];
            }
        }
    };
    if (bias_rows) bias_request(bvs[0], 0);
#pragma unroll
    for (int i = 0; i < FM; i++) {
        if (bias_rows && i + 1 < FM) bias_request(bvs[(i + 1) & 1], i + 1);
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int gm = m0 + wm * TM + (lq * 4 + r) * FM + i;
            float v[FN];
#pragma unroll
            for (int j = 0; j < FN; j++) {
                float x = acc[(j >> 2) * HALF + i * 4 + (j & 3)][r] + (bias_rows ? bvs[i & 1][r][j] : bcol[j]);
                if (p.relu) x = x > 0.f ? x : 0.f;
                v[j] = poisoned ? __builtin_nanf("") : x;
            }
            float* dst = C + (long)gm * p.ldc + gn;
            floatx4 o0 = {v[0], v[1], v[2], v[3]}, o1 = {v[4], v[5], v[6], v[7]};
            *reinterpret_cast<floatx4*>(dst) = o0;
            *reinterpret_cast<floatx4*>(dst + 4) = o1;
        }
    }
}

// ---- host side -----------------------------------------------------------------------------
static inline long round_up(long v, long q) { return (v + q - 1) / q * q; }

bool gemm_h16_applicable(const nzhip_gemm_desc& d) {
    // Worth it when each operand element is re-read by many tiles, i.e. when the GEMM does far
    // more work per operand byte than the extra rounding pass moves. Measured on MI355X
    // (microseconds, fused / two-pass): 3072^3 136 / 102, 4096^3 197 / 163, 4096x4096x1024 60 / 52,
    // but 2048^3 44 / 53, 4096x1024x4096 67 / 77, 4096x256x4096 30 / 36, 8192x512x8192 160 / 168 (short contractions leave
    // the rounding pass and the C stores nothing to hide behind). Shapes that are not whole
    // 256x256x32 tiles take the fused kernel's predicated instance, which is much slower, so the
    // threshold is lower for them: 2500^3 101 / 68, 5000x1000x5000 156 / 94, 2000^3 56 / 55.
    if (d.M < 512 || d.N < 512 || d.K < 768) return false;
    const double flops = 2.0 * d.M * d.N * d.K;
    const double cvt_bytes = 6.0 * ((double)d.M * d.K + (double)d.N * d.K);
    const bool whole_tiles = d.M % 256 == 0 && d.N % 256 == 0 && d.K % 32 == 0 && d.lda % 4 == 0 && d.ldb % 4 == 0 &&
                             d.ldc % 4 == 0;
    // (whole tiles, fused / two-pass: 2048^3 38 / 45 and 2048x2048x4096 67 / 74 at a ratio of 341, but 2304^3 62 / 50 at 384,
    // 3072x2048x2048 55 / 47 at 410, 2560^3 71 / 55 at 427, 4096x2048x4096 118 / 92 and 2048x4096x3072 94 / 73 at 455)
    return flops / cvt_bytes >= (whole_tiles ? 360.0 : 300.0);
}

// Host-side bookkeeping of the bounded waits: which stream the products enqueued since the last look went to,
// how many time-outs had been seen by then, and whether the route has been given up.
static std::mutex g_coop_mu;
static unsigned g_coop_pending = 0;              // single-kernel products enqueued since the last look
static hipStream_t g_coop_stream = nullptr;      // the stream they all went to ...
static bool g_coop_mixed = false;                // ... unless they went to several
static unsigned g_coop_seen = 0;                 // value of g_coop_timeouts at the last look
static std::atomic<bool> g_coop_off{false};
static std::atomic<unsigned> g_coop_spin_limit{200000};   // x (16 sleeps + one read): a few hundred ms
static std::atomic<int> g_coop_mute{0};                   // test hook, see CoopArgs::mute

// The single-kernel route wants one unbatched product of whole 16 x 16 tile blocks and whole panels, 16-byte
// accesses everywhere, at least two stages to overlap, and a device on which a wave of 256 workgroups is
// resident at once (one workgroup per CU).
bool gemm_h16_coop_applicable(const nzhip_gemm_desc& d) {
    if (g_coop_off.load(std::memory_order_relaxed)) return false;
    constexpr int64_t BLOCK = (int64_t)COOP_SB * 256, PANEL = (int64_t)COOP_KP * CVT_K;
    if (d.batch_n * d.batch_c != 1) return false;
    if (d.M < BLOCK || d.N < BLOCK || d.M % BLOCK || d.N % BLOCK || d.K % PANEL) return false;
    const int64_t waves = (d.M / BLOCK) * (d.N / BLOCK), panels = d.K / PANEL;
    if (waves * panels < 2 || waves > 16384) return false;
    if (d.lda % 4 || d.ldb % 4 || d.ldc % 4) return false;
    if ((reinterpret_cast<uintptr_t>(d.A) | reinterpret_cast<uintptr_t>(d.B) | reinterpret_cast<uintptr_t>(d.C)) & 15) return false;
    return device_cu_count() == COOP_WG;
}

int gemm_h16_coop_dispatch(const nzhip_gemm_desc& d, hipStream_t s) {
    const long Mp = d.M, Np = d.N, Kp = d.K;
    const bool a_kc = d.a_layout != NZHIP_LAYOUT_TRANS, b_kc = d.b_layout == NZHIP_LAYOUT_TRANS;
    const size_t a_elems = (size_t)Mp * Kp, b_elems = (size_t)Np * Kp;
    const int nkt = (int)(Kp / CVT_K), panels = nkt / COOP_KP;
    const int sm = (int)(Mp / (COOP_SB * 256)), sn = (int)(Np / (COOP_SB * 256)), waves = sm * sn;
    const int n_flags = waves * panels + 1;                             // stage counters + the launch's time-out count
    const size_t img_bytes = (a_elems + b_elems) * sizeof(_Float16);
    char* ws = nullptr;
    if (int rc = workspace_alloc(reinterpret_cast<void**>(&ws), img_bytes + (size_t)n_flags * sizeof(unsigned), s)) return rc;
    _Float16* Ah = reinterpret_cast<_Float16*>(ws);
    _Float16* Bh = Ah + a_elems;
    unsigned* flags = reinterpret_cast<unsigned*>(ws + img_bytes);

    auto operand = [&](_Float16* dst, const float* src, long R, long ld, int fr) {
        CvtOperand o;
        o.dst = dst; o.src = src; o.R = (int)R; o.ld = ld;
        o.src_batch = 0; o.dst_batch = 0; o.vec = 1; o.fr = fr;
        return o;
    };
    const CvtOperand oa = operand(Ah, d.A, d.M, d.lda, 4), ob = operand(Bh, d.B, d.N, d.ldb, 8);
    CoopArgs a;
    H16Args& g = a.g;
    g.A = Ah; g.B = Bh; g.C = d.C; g.bias = d.bias;
    g.M = (int)d.M; g.N = (int)d.N; g.Kp = (int)Kp; g.ldc = d.ldc;
    g.batch_c = 1; g.batch = 1; g.a_batch = g.b_batch = 0;
    g.a_bcast_n = g.a_bcast_c = g.b_bcast_n = g.b_bcast_c = 1;
    g.a_cn = g.b_cn = 1;
    g.c_sn = g.c_sc = g.bias_sn = g.bias_sc = 0;
    g.bias_sm = d.bias_stride_row; g.bias_sk = d.bias_stride_col;
    g.relu = d.activation == NZHIP_ACT_RELU;
    g.tiles_m = (int)(Mp / 256); g.tiles_n = (int)(Np / 256); g.group_m = 4;
    a.srcA = d.A; a.srcB = d.B; a.lda = d.lda; a.ldb = d.ldb;
    a.flags = flags; a.sn = sn; a.waves = waves; a.panels = panels;
    a.spin_limit = g_coop_spin_limit.load(std::memory_order_relaxed);
    a.mute = g_coop_mute.load(std::memory_order_relaxed);

    // stage (0, 0): the first 16 row blocks of both operands over the first panel; also clears the counters
    dim3 pgrid((unsigned)COOP_KP, (unsigned)(2 * COOP_SB), 1);
    constexpr size_t lds_bytes = 4 * (256 + 256) * 64 + 2 * CVT_BLOCK_BYTES;   // ring + fp32 staging = all 160 KiB
    int rc = NZHIP_OK;
#define NZHIP_COOP(AK, BK)                                                                                         \
    do {                                                                                                           \
        hipLaunchKernelGGL((coop_prologue_kernel<AK, BK>), pgrid, dim3(256), 0, s, oa, ob, COOP_SB, (int)d.K, nkt, \
                           flags, n_flags);                                                                        \
        auto kfn = gemm_h16c_kernel<AK, BK>;                                                                       \
        rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kfn), (int)lds_bytes, "hipFuncSetAttribute(gemm_h16c)"); \
        if (rc == NZHIP_OK) hipLaunchKernelGGL(kfn, dim3((unsigned)(waves * COOP_WG)), dim3(512), lds_bytes, s, a); \
    } while (0)
    if (a_kc && b_kc) NZHIP_COOP(true, true);
    else if (a_kc) NZHIP_COOP(true, false);
    else if (b_kc) NZHIP_COOP(false, true);
    else NZHIP_COOP(false, false);
#undef NZHIP_COOP
    if (rc == NZHIP_OK) {
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) rc = set_hip_error(e, "gemm_h16c kernel launch");
    }
    {
        std::lock_guard<std::mutex> lock(g_coop_mu);
        if (g_coop_pending && g_coop_stream != s) g_coop_mixed = true;
        g_coop_stream = s;
        g_coop_pending++;
    }
    int rc2 = workspace_free(ws, s);
    return rc ? rc : rc2;
}

int gemm_h16_coop_check(hipStream_t drained, bool whole_device) {
    std::lock_guard<std::mutex> lock(g_coop_mu);
    if (!g_coop_pending) return NZHIP_OK;
    if (!whole_device && (g_coop_mixed || g_coop_stream != drained)) return NZHIP_OK;   // may still be running
    unsigned count = 0;
    hipError_t e = hipMemcpyFromSymbol(&count, HIP_SYMBOL(g_coop_timeouts), sizeof(unsigned));
    if (e != hipSuccess) return set_hip_error(e, "hipMemcpyFromSymbol(g_coop_timeouts)");
    g_coop_pending = 0;
    g_coop_mixed = false;
    if (count == g_coop_seen) return NZHIP_OK;
    const unsigned fresh = count - g_coop_seen;
    g_coop_seen = count;
    g_coop_off.store(true, std::memory_order_relaxed);
    return set_error(NZHIP_E_TIMEOUT,
                     "nzhip_gemm: %u bounded waits of the single-kernel route ran out (is the device shared?): that product "
                     "holds NaN in every tile stored after the first of them; this process uses the two-kernel route from now on",
                     fresh);
}

int gemm_h16_coop_reset(unsigned inject) {
    std::lock_guard<std::mutex> lock(g_coop_mu);
    hipError_t e = hipDeviceSynchronize();
    if (e != hipSuccess) return set_hip_error(e, "hipDeviceSynchronize");
    unsigned count = 0;
    e = hipMemcpyFromSymbol(&count, HIP_SYMBOL(g_coop_timeouts), sizeof(unsigned));
    if (e != hipSuccess) return set_hip_error(e, "hipMemcpyFromSymbol(g_coop_timeouts)");
    if (inject) {
        count += inject;
        e = hipMemcpyToSymbol(HIP_SYMBOL(g_coop_timeouts), &count, sizeof(unsigned));
        if (e != hipSuccess) return set_hip_error(e, "hipMemcpyToSymbol(g_coop_timeouts)");
    } else {
        count = 0;
        e = hipMemcpyToSymbol(HIP_SYMBOL(g_coop_timeouts), &count, sizeof(unsigned));
        if (e != hipSuccess) return set_hip_error(e, "hipMemcpyToSymbol(g_coop_timeouts)");
        g_coop_seen = 0;
        g_coop_pending = 0;
        g_coop_mixed = false;
        g_coop_off.store(false, std::memory_order_relaxed);
    }
    return NZHIP_OK;
}

void gemm_h16_coop_test_mode(unsigned spin_limit, int mute) {
    g_coop_spin_limit.store(spin_limit ? spin_limit : 200000u, std::memory_order_relaxed);
    g_coop_mute.store(mute, std::memory_order_relaxed);
}

int gemm_h16_coop_timeouts(unsigned* count) {
    hipError_t e = hipMemcpyFromSymbol(count, HIP_SYMBOL(g_coop_timeouts), sizeof(unsigned));
    return e == hipSuccess ? NZHIP_OK : set_hip_error(e, "hipMemcpyFromSymbol(g_coop_timeouts)");
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

    // The image of A comes from the pooled workspace. The image of B may belong to a prepared-operand handle
    // (nzhip_gemm_prepared_b): its layout does not depend on the kernel variant beyond the MFMA block height, so an
    // image built by an earlier call with the same operand is used as it is and B's rounding pass is skipped.
    _Float16* Ah = nullptr;
    if (int rc = workspace_alloc(reinterpret_cast<void**>(&Ah), a_total * sizeof(_Float16), s)) return rc;
    uint64_t key[PREPARED_KEY_WORDS] = {};
    key[0] = 4u | ((uint64_t)blk << 8) | ((uint64_t)fr_b << 16) | ((uint64_t)(b_trans ? 1 : 0) << 24);
    key[1] = reinterpret_cast<uintptr_t>(d.B);
    key[2] = (uint64_t)d.N; key[3] = (uint64_t)d.K; key[4] = (uint64_t)d.ldb;
    key[5] = (uint64_t)b_n; key[6] = (uint64_t)b_c; key[7] = (uint64_t)d.b_stride_n; key[8] = (uint64_t)d.b_stride_c;
    ImageLease b_lease;
    if (int rc = image_acquire(PREPARED_GEMM_B, key, b_total * sizeof(_Float16), s, &b_lease)) {
        workspace_free(Ah, s);
        return rc;
    }
    _Float16* Bh = static_cast<_Float16*>(b_lease.ptr);

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
    int rc;
    if (b_lease.fill && a_n == 1 && b_n == 1 && a_c == b_c && (Mp + Np) / CVT_ROWS <= 65535) {
        rc = convert_pair(fr_a, fr_b, blk);
    } else {
        rc = convert(Ah, d.A, d.M, Mp, !a_trans, d.lda, a_n, a_c, d.a_stride_n, d.a_stride_c, a_elems, fr_a, blk);
        if (rc == NZHIP_OK && b_lease.fill)
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
    int rc2 = workspace_free(Ah, s);
    const int rc3 = image_release(b_lease, s, rc == NZHIP_OK);
    if (!rc2) rc2 = rc3;
    return rc ? rc : rc2;
}

}  // namespace nzhip
