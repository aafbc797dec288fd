// Conv2d forward: the Model::Conv2d graph of the reference (src/Model.cu:244-263:
// Img2Col -> MatMul -> Bias -> Col2Img [-> ReLU]) as one call.
#include <hip/hip_runtime.h>

#include <type_traits>

#include <cstdlib>

#include "nzhip_internal.h"

namespace nzhip {

typedef float floatx4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float round_f16(float x) { return (float)(_Float16)x; }

// v when keep, +0 otherwise, as a bit mask: keeps the producing load unconditional (a select on
// the value invites the compiler to sink the load into a branch, which then has to wait for it
// immediately and serialises the prefetch).
__device__ __forceinline__ float keep_or_zero(float v, bool keep) {
    return __builtin_bit_cast(float, __builtin_bit_cast(unsigned, v) & (keep ? 0xffffffffu : 0u));
}

// ---- direct route: 3x3, stride 1, pad 1, few output channels -------------------------------
// With a handful of output channels the product has K = C*9 and N = O <= 4: far too small for
// MFMA to matter, the op is a pure stream (each input element needed by 9 outputs). Every lane
// owns 4 adjacent output pixels of ROWS consecutive rows, walks down the image keeping the
// partial sums of the three output rows an input row contributes to, and reads each input row
// once: one 16-byte load plus the two halo pixels (which hit in L1, they are the neighbour
// lanes' 16 bytes). Operands are rounded to fp16 and accumulated in fp32 by FMA in the
// reference's k order q = c*9 + r*3 + s, so the result equals the k-ascending fp32 sum of the
// im2col + GEMM graph bit for bit. Output stores are 16-byte and contiguous along w.
constexpr int DC_ROWS = 4;         // output rows per wave
constexpr int DC_MAX_C = 8;        // input channels held in the rolling window
constexpr int DC_MAX_O = 4;

// Workgroups are dealt to the eight XCDs round-robin by their linear index, and every XCD has an L2 of
// its own. This renumbers them so that each XCD works on one contiguous run of the (x, y, z) grid in
// x-fastest order: neighbouring tiles, which share halo rows and the memory lines of their edge
// columns, then meet in one L2 instead of fetching those lines twice.
__device__ __forceinline__ void xcd_contiguous_block(int& bx, int& by, int& bz) {
    const long gx = gridDim.x, gy = gridDim.y;
    const long total = gx * gy * gridDim.z;
    const long lin = blockIdx.x + gx * (blockIdx.y + gy * blockIdx.z);
    const long xcd = lin & 7, q = lin >> 3;
    const long rem = total & 7;
    const long unit = xcd * (total >> 3) + (xcd < rem ? xcd : rem) + q;
    bx = (int)(unit % gx);
    by = (int)((unit / gx) % gy);
    bz = (int)(unit / (gx * gy));
}

// The same with z (the image) fastest inside an XCD's run: the XCD then works on one stretch of the (x, y) grid for ALL
// images, so whatever the images share per tile -- a per-pixel bias -- is fetched into its L2 once instead of once per image.
__device__ __forceinline__ void xcd_contiguous_block_z_fastest(int& bx, int& by, int& bz) {
    const long gx = gridDim.x, gz = gridDim.z;
    const long total = gx * gridDim.y * gz;
    const long lin = blockIdx.x + gx * (blockIdx.y + (long)gridDim.y * blockIdx.z);
    const long xcd = lin & 7, q = lin >> 3;
    const long rem = total & 7;
    const long unit = xcd * (total >> 3) + (xcd < rem ? xcd : rem) + q;
    bz = (int)(unit % gz);
    bx = (int)((unit / gz) % gx);
    by = (int)(unit / (gz * gx));
}

// O_T: output channels per thread; C_T: compile-time input-channel count (0 = runtime loop);
// VEC: W % 4 == 0 and 16-byte aligned tensors, so every lane's 4 pixels are inside the row and
// move as one 16-byte access.
template <int O_T, int C_T, bool VEC>
__global__ __launch_bounds__(256) void conv3x3_direct_kernel(float* __restrict__ y, const float* __restrict__ x,
                                                             const float* __restrict__ w_ref,
                                                             const float* __restrict__ bias, int C_rt, int H, int W,
                                                             int O, long w_batch_stride, long bias_sp, long bias_sc,
                                                             int relu) {
    __shared__ _Float16 wsm[DC_MAX_C * 9 * DC_MAX_O];
    const int C = C_T ? C_T : C_rt;
    int bx, by, b;
    xcd_contiguous_block(bx, by, b);
    const float* wb = w_ref + (long)b * w_batch_stride;
    for (int i = threadIdx.x; i < C * 9 * O; i += 256) wsm[i] = (_Float16)wb[i];     // [q][o], RNE
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int w0 = (bx * 64 + lane) * 4;
    const int h0 = (by * 4 + wave) * DC_ROWS;
    if (w0 >= W || h0 >= H) return;
    const float* xb = x + (long)b * C * H * W;
    float* yb = y + (long)b * O * H * W;

    float acc[DC_ROWS][O_T][4];
#pragma unroll
    for (int j = 0; j < DC_ROWS; j++)
#pragma unroll
        for (int o = 0; o < O_T; o++)
#pragma unroll
            for (int e = 0; e < 4; e++) acc[j][o][e] = 0.f;

    // halo columns, clamped so the address is always inside the row; the value is zeroed afterwards
    const int wl = w0 > 0 ? w0 - 1 : 0, wr = w0 + 4 < W ? w0 + 4 : W - 1;
    const bool has_l = w0 > 0, has_r = w0 + 4 < W;

    // load one input row of channel c (columns w0-1 .. w0+4) as raw fp32
    auto load_row = [&](int c, int t, float (&m)[6]) {
        const int hi = h0 - 1 + t;
        const bool row_ok = hi >= 0 && hi < H;                           // wave-uniform
        const float* row = xb + (long)c * H * W + (long)(row_ok ? hi : 0) * W;
        if (VEC) {
            const floatx4 q = *reinterpret_cast<const floatx4*>(row + w0);
            m[1] = q[0]; m[2] = q[1]; m[3] = q[2]; m[4] = q[3];
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int we = w0 + e < W ? w0 + e : W - 1;
                const float q = row[we];
                m[1 + e] = w0 + e < W ? q : 0.f;
            }
        }
        const float ql = row[wl], qr = row[wr];
        m[0] = keep_or_zero(ql, has_l);
        m[5] = keep_or_zero(qr, has_r);
    };
    // Round the row to fp16 (RNE) and add its contribution. Input row t feeds output row
    // j = t - r (r = 0..2); for a fixed output row, r = t - j ascends with t, so the accumulation
    // order is the reference's q = c*9 + r*3 + s.
    auto consume_row = [&](int c, int t, const float (&m)[6]) {
        const int hi = h0 - 1 + t;
        const bool row_ok = hi >= 0 && hi < H;
        _Float16 v[6];
#pragma unroll
        for (int e = 0; e < 6; e++) v[e] = row_ok ? (_Float16)m[e] : (_Float16)0.f;
#pragma unroll
        for (int r = 0; r < 3; r++) {
            const int j = t - r;
            if (j < 0 || j >= DC_ROWS) continue;
#pragma unroll
            for (int s = 0; s < 3; s++) {
#pragma unroll
                for (int o = 0; o < O_T; o++) {
                    const _Float16 wv = wsm[(c * 9 + r * 3 + s) * O + o];
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        acc[j][o][e] = __builtin_fmaf((float)v[e + s], (float)wv, acc[j][o][e]);
                }
            }
        }
    };
    if constexpr (C_T > 0 && C_T <= 3) {
        // few channels: request every row of every channel before touching any, so a wave pays
        // the memory latency once
        float raw[C_T][DC_ROWS + 2][6];
#pragma unroll
        for (int c = 0; c < C_T; c++)
#pragma unroll
            for (int t = 0; t < DC_ROWS + 2; t++) load_row(c, t, raw[c][t]);
#pragma unroll
        for (int c = 0; c < C_T; c++)
#pragma unroll
            for (int t = 0; t < DC_ROWS + 2; t++) consume_row(c, t, raw[c][t]);
    } else {
        for (int c = 0; c < C; c++) {
            float raw[DC_ROWS + 2][6];
#pragma unroll
            for (int t = 0; t < DC_ROWS + 2; t++) load_row(c, t, raw[t]);
#pragma unroll
            for (int t = 0; t < DC_ROWS + 2; t++) consume_row(c, t, raw[t]);
        }
    }

#pragma unroll
    for (int j = 0; j < DC_ROWS; j++) {
        const int ho = h0 + j;
        if (ho >= H) continue;
#pragma unroll
        for (int o = 0; o < O_T; o++) {
            float out[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                float a = acc[j][o][e];
                if (bias && (VEC || w0 + e < W)) a += bias[((long)ho * W + w0 + e) * bias_sp + (long)o * bias_sc];
                if (relu) a = a > 0.f ? a : 0.f;
                out[e] = a;
            }
            float* dst = yb + ((long)o * H + ho) * W + w0;
            if (VEC) {
                floatx4 ov = {out[0], out[1], out[2], out[3]};
                *reinterpret_cast<floatx4*>(dst) = ov;
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (w0 + e < W) dst[e] = out[e];
            }
        }
    }
}

// ---- streaming variant of the direct route (C <= 4, O <= 2, 16-byte aligned rows) ----------
// A wave owns a strip of 256 columns x ST_ROWS output rows and walks DOWN it: every input row
// is requested once, ST_AHEAD rows ahead of its use, rounded to fp16 once, and kept in a
// rolling window of three rows per channel; as soon as a row arrives, the output row above it
// is complete and is computed in the reference's k order (c, r, s) and stored. Loads of later
// rows are in flight while the FMAs of the current row run, so memory and VALU time overlap
// inside every wave instead of relying on other waves being out of phase.
// A lane's two halo columns are its neighbours' pixels: they come over the wave (DPP shift by one
// lane) after rounding; only the first and the last lane of a wave read theirs from memory, with
// one extra 4-byte request per row and channel that every lane issues (the others re-read a word
// of their own quad). PIX_BIAS: the bias varies per pixel and travels with the row ring; otherwise
// it is absent or per channel and is fetched once.
constexpr int ST_ROWS = 16, ST_AHEAD = 3;         // ST_AHEAD: a multiple of 3 (the window depth)

// value of `v` in lane - 1 (lane 0 keeps its own)
__device__ __forceinline__ float from_lane_below(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v),
                                                                 0x138 /* wave_shr:1 */, 0xf, 0xf, false));
}
// value of `v` in lane + 1 (lane 63 keeps its own)
__device__ __forceinline__ float from_lane_above(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v),
                                                                 0x130 /* wave_shl:1 */, 0xf, 0xf, false));
}

// PIX_BIAS: 0 none or per channel; 1 per pixel with any strides; 2 per pixel in the layout of the
// reference's Bias node ([pixel][channel], 16-byte aligned), where a lane's 4 pixels x O_T channels are one
// contiguous run fetched with 16-byte loads.
template <int O_T, int C_T, int PIX_BIAS>
__global__ __launch_bounds__(256) void conv3x3_stream_kernel(float* __restrict__ y, const float* __restrict__ x,
                                                             const float* __restrict__ w_ref,
                                                             const float* __restrict__ bias, int H, int W,
                                                             long w_batch_stride, long bias_sp, long bias_sc,
                                                             int relu) {
    __shared__ float wsm[C_T * 9 * O_T];
    int bx, by, b;
    xcd_contiguous_block(bx, by, b);
    const float* wb = w_ref + (long)b * w_batch_stride;
    static_assert(C_T * 9 * O_T <= 128, "one weight per thread");
    // requested now, parked in LDS after the first input rows have been requested (the rows then do not
    // queue up behind the round trip of the weights)
    const float w_mine = threadIdx.x < C_T * 9 * O_T ? wb[threadIdx.x] : 0.f;
    auto park_weights = [&]() {
        if (threadIdx.x < C_T * 9 * O_T) wsm[threadIdx.x] = round_f16(w_mine);   // [q][o]
        __syncthreads();
    };

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int strip = by * 4 + wave;
    const int h0 = strip * ST_ROWS;
    if (h0 >= H) {                                               // a whole wave with nothing to do but the workgroup's one barrier
        park_weights();
        return;
    }
    // Lanes past the last column stay in the walk (the barrier in park_weights() must not sit in a branch that
    // only some lanes of a wave take): they work on the image's last quad of columns and store nothing.
    const bool active = (bx * 64 + lane) * 4 < W;
    const int w0 = active ? (bx * 64 + lane) * 4 : W - 4;
    const float* xb = x + (long)b * C_T * H * W;
    float* yb = y + (long)b * O_T * H * W;
    const long plane = (long)H * W;
    const bool has_l = w0 > 0, has_r = w0 + 4 < W;
    // column of the extra request: left halo for the first lane, right halo for the last, else own quad
    const int wx = lane == 0 ? (has_l ? w0 - 1 : w0) : (lane == 63 && has_r ? w0 + 4 : w0);
    const int rows = (H - h0) < ST_ROWS ? (H - h0) : ST_ROWS;   // output rows of this strip
    const int T = rows + 2;                                      // input rows h0-1 .. h0+rows
    // Odd strips walk upwards. A strip shares its first and its last input rows with its neighbours;
    // with alternating directions both neighbours touch a shared row at the same moment (both at the
    // start, or both at the end of their walk), so the second request finds it in L2. Walking all
    // strips downwards puts a whole strip's duration between the two uses and the row comes from
    // memory twice. The walk is instantiated once per direction and a wave runs one of the two.
    const bool rev = (strip & 1) != 0;
    auto walk = [&](auto upwards) {
    constexpr bool UP = decltype(upwards)::value;
    const int row_first = UP ? h0 + rows : h0 - 1, row_step = UP ? -1 : 1;
    auto out_row = [&](int t) { return UP ? h0 + rows + 1 - t : h0 + t - 2; };   // completed by step t >= 2
    float raw[ST_AHEAD][C_T][5];                                 // rows in flight (t % ST_AHEAD): own quad + extra word
    float braw[ST_AHEAD][O_T][4];                                // per-pixel bias of the output row each completes
    float win[3][C_T][6];                                        // rounded rows t-2, t-1, t (t % 3)
    float bch[O_T];                                              // per-channel bias
#pragma unroll
    for (int o = 0; o < O_T; o++) bch[o] = (!PIX_BIAS && bias) ? bias[(long)o * bias_sc] : 0.f;

    // Requests are unconditional (rows beyond the image read row 0); what must be zero is masked
    // when the row is consumed, so nothing waits at request time.
    auto row_in_image = [&](int t) { const int hi = row_first + t * row_step; return t < T && hi >= 0 && hi < H; };
    auto request = [&](int t, float (&dst)[C_T][5], float (&bdst)[O_T][4]) {
        const float* row = xb + (long)(row_in_image(t) ? row_first + t * row_step : 0) * W;
        if (PIX_BIAS) {
            // the bias of the output row a step completes travels with that step's input row, so its
            // wait never drains the rows requested after it
            const int hb = (t >= 2 && t < T) ? out_row(t) : h0;
            if (PIX_BIAS == 2) {
                const floatx4* run = reinterpret_cast<const floatx4*>(bias + ((long)hb * W + w0) * O_T);
#pragma unroll
                for (int k = 0; k < O_T; k++) {
                    const floatx4 v = run[k];                    // elements 4k..4k+3 of the run: (pixel, channel) = (i / O_T, i % O_T)
#pragma unroll
                    for (int j = 0; j < 4; j++) bdst[(4 * k + j) % O_T][(4 * k + j) / O_T] = v[j];
                }
            } else {
#pragma unroll
                for (int o = 0; o < O_T; o++)
#pragma unroll
                    for (int e = 0; e < 4; e++) bdst[o][e] = bias[((long)hb * W + w0 + e) * bias_sp + (long)o * bias_sc];
            }
        }
#pragma unroll
        for (int c = 0; c < C_T; c++) {
            const floatx4 q = *reinterpret_cast<const floatx4*>(row + c * plane + w0);
            dst[c][0] = q[0];
            dst[c][1] = q[1];
            dst[c][2] = q[2];
            dst[c][3] = q[3];
            dst[c][4] = row[c * plane + wx];
        }
    };

#pragma unroll
    for (int t = 0; t < ST_AHEAD; t++) request(t, raw[t], braw[t]);
    park_weights();

    static_assert(ST_AHEAD % 3 == 0, "the request ring must be a whole number of windows");
    for (int t0 = 0; t0 < T; t0 += ST_AHEAD) {
#pragma unroll
        for (int u = 0; u < ST_AHEAD; u++) {
            const int t = t0 + u;                                // t % ST_AHEAD == u, and t % 3 == u % 3
            const int wu = u % 3;
            if (t >= T) break;
            const bool in_img = row_in_image(t);
#pragma unroll
            for (int c = 0; c < C_T; c++) {
                float r5[5];
#pragma unroll
                for (int e = 0; e < 5; e++) {
                    // Opaque use: pins the rounding (and therefore the wait for the load) HERE, three
                    // rows after the request; otherwise the compiler moves the conversion up to the
                    // load and the wave waits for every row as soon as it has asked for it.
                    float v = raw[u][c][e];
                    asm volatile("" : "+v"(v));
                    r5[e] = in_img ? round_f16(v) : 0.f;
                }
                const float below = from_lane_below(r5[3]), above = from_lane_above(r5[0]);
                win[wu][c][0] = has_l ? (lane == 0 ? r5[4] : below) : 0.f;
#pragma unroll
                for (int e = 0; e < 4; e++) win[wu][c][1 + e] = r5[e];
                win[wu][c][5] = has_r ? (lane == 63 ? r5[4] : above) : 0.f;
            }
            float bnow[O_T][4];
#pragma unroll
            for (int o = 0; o < O_T; o++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    bnow[o][e] = PIX_BIAS ? braw[u][o][e] : bch[o];
                    if (PIX_BIAS) asm volatile("" : "+v"(bnow[o][e]));
                }
            request(t + ST_AHEAD, raw[u], braw[u]);              // slot u is free again
            if (t < 2) continue;
            const int ho = out_row(t);                           // output row fed by the rows of steps t-2, t-1, t
            float acc[O_T][4];
#pragma unroll
            for (int o = 0; o < O_T; o++)
#pragma unroll
                for (int e = 0; e < 4; e++) acc[o][e] = 0.f;
            // Filter row r meets the input row of step t-2+r (walking down) or t-r (walking up), which
            // lives in slot (step % 3); the sum runs over c, r, s in ascending order either way.
#pragma unroll
            for (int c = 0; c < C_T; c++)
#pragma unroll
                for (int r = 0; r < 3; r++) {
                    const int slot = UP ? (wu + 3 - r) % 3 : (wu + 1 + r) % 3;
#pragma unroll
                    for (int s2 = 0; s2 < 3; s2++)
#pragma unroll
                        for (int o = 0; o < O_T; o++) {
                            const float wv = wsm[(c * 9 + r * 3 + s2) * O_T + o];
#pragma unroll
                            for (int e = 0; e < 4; e++) acc[o][e] = __builtin_fmaf(win[slot][c][e + s2], wv, acc[o][e]);
                        }
                }
#pragma unroll
            for (int o = 0; o < O_T; o++) {
                floatx4 ov;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float a = acc[o][e] + bnow[o][e];
                    if (relu) a = a > 0.f ? a : 0.f;
                    ov[e] = a;
                }
                if (active) *reinterpret_cast<floatx4*>(yb + ((long)o * H + ho) * W + w0) = ov;
            }
        }
    }
    };
    if (rev) walk(std::true_type{});
    else walk(std::false_type{});
}

static bool conv_direct_applicable(size_t C, size_t O, size_t K_h, size_t K_w, size_t stride, size_t pad) {
    return K_h == 3 && K_w == 3 && stride == 1 && pad == 1 && C <= DC_MAX_C && O <= DC_MAX_O && O >= 1;
}

static int conv_direct(float* y, const float* x, const float* w_ref, const float* bias, size_t N, size_t C, size_t H,
                       size_t W, size_t O, size_t w_batch, int64_t bias_sp, int64_t bias_sc, int act, hipStream_t s) {
    if (N > 65535) return set_error(NZHIP_E_UNSUPPORTED, "nzhip_conv2d_forward: batch above 65535");
    const int vec = (W % 4 == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0) && ((reinterpret_cast<uintptr_t>(y) & 15) == 0);
    dim3 grid((unsigned)((W + 255) / 256), (unsigned)((H + 4 * DC_ROWS - 1) / (4 * DC_ROWS)), (unsigned)N);
    const long wbs = w_batch > 1 ? (long)(C * 9 * O) : 0;
    if (vec && C <= 4 && O <= 2 && H >= 8) {
        dim3 sgrid((unsigned)((W + 255) / 256), (unsigned)((H + 4 * ST_ROWS - 1) / (4 * ST_ROWS)), (unsigned)N);
        const bool pixb = bias && bias_sp != 0;
        // the reference's Bias node: [pixel][channel], so the bias of a lane's 4 pixels is one aligned run
        const bool pixrun = pixb && bias_sp == (int64_t)O && bias_sc == 1 && (reinterpret_cast<uintptr_t>(bias) & 15) == 0;
#define NZHIP_ST(OT, CT)                                                                                             \
    do {                                                                                                             \
        if (pixrun)                                                                                                  \
            hipLaunchKernelGGL((conv3x3_stream_kernel<OT, CT, 2>), sgrid, dim3(256), 0, s, y, x, w_ref, bias, (int)H,  \
                               (int)W, wbs, (long)bias_sp, (long)bias_sc, act == NZHIP_ACT_RELU);                   \
        else if (pixb)                                                                                               \
            hipLaunchKernelGGL((conv3x3_stream_kernel<OT, CT, 1>), sgrid, dim3(256), 0, s, y, x, w_ref, bias, (int)H,  \
                               (int)W, wbs, (long)bias_sp, (long)bias_sc, act == NZHIP_ACT_RELU);                   \
        else                                                                                                         \
            hipLaunchKernelGGL((conv3x3_stream_kernel<OT, CT, 0>), sgrid, dim3(256), 0, s, y, x, w_ref, bias, (int)H,  \
                               (int)W, wbs, (long)bias_sp, (long)bias_sc, act == NZHIP_ACT_RELU);                   \
    } while (0)
        switch ((int)(O * 10 + C)) {
            case 11: NZHIP_ST(1, 1); break;
            case 12: NZHIP_ST(1, 2); break;
            case 13: NZHIP_ST(1, 3); break;
            case 14: NZHIP_ST(1, 4); break;
            case 21: NZHIP_ST(2, 1); break;
            case 22: NZHIP_ST(2, 2); break;
            case 23: NZHIP_ST(2, 3); break;
            default: NZHIP_ST(2, 4); break;
        }
#undef NZHIP_ST
        hipError_t e = hipGetLastError();
        return e == hipSuccess ? NZHIP_OK : set_hip_error(e, "conv3x3_stream_kernel launch");
    }
#define NZHIP_DC(OT, CT, V)                                                                                     \
    hipLaunchKernelGGL((conv3x3_direct_kernel<OT, CT, V>), grid, dim3(256), 0, s, y, x, w_ref, bias, (int)C, (int)H, \
                       (int)W, (int)O, wbs, (long)bias_sp, (long)bias_sc, act == NZHIP_ACT_RELU)
#define NZHIP_DC_O(CT, V)            \
    switch (O) {                     \
        case 1: NZHIP_DC(1, CT, V); break; \
        case 2: NZHIP_DC(2, CT, V); break; \
        case 3: NZHIP_DC(3, CT, V); break; \
        default: NZHIP_DC(4, CT, V); break; \
    }
    if (vec) {
        if (C == 3) { NZHIP_DC_O(3, true) } else if (C == 1) { NZHIP_DC_O(1, true) } else { NZHIP_DC_O(0, true) }
    } else {
        NZHIP_DC_O(0, false)
    }
#undef NZHIP_DC_O
#undef NZHIP_DC
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? NZHIP_OK : set_hip_error(e, "conv3x3_direct_kernel launch");
}

// ---- implicit-GEMM route: stride 1, many channels ------------------------------------------
// No column matrix exists anywhere. A workgroup owns an 8 x 32 patch of output pixels of one
// image and 128 output channels, and walks the input channels 16 at a time. Per chunk it
//   * stages the (8+KH-1) x (32+KW-1) x 16 input halo ONCE: fp32 NCHW -> fp16 (RNE),
//     channel-last in LDS, so the 8 consecutive k a lane feeds to an MFMA are the 8
//     consecutive channels of one pixel (one 16-byte LDS read), for every filter tap;
//   * pulls the matching weight slab (pre-rounded to fp16 and pre-arranged by a small
//     pre-pass into the exact LDS image, 16-byte row pad included) with direct-to-LDS loads;
//   * issues KH*KW k-steps of v_mfma_f32_32x32x16_f16: weights are the row operand, pixels the
//     column operand, so lanes map to adjacent pixels and the NCHW store (the reference's
//     col2im transpose, src/OperationKernels.cu:1364-1376) is contiguous, with bias and ReLU
//     applied on the way out.
// k runs in the order (channel chunk, tap, channel) instead of the reference's
// q = c*KH*KW + r*KW + s; only the fp32 summation order differs.
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int IG_PIX = 256, IG_CC = 16;

// TW: width of the pixel patch (32 or 64); its height is 256 / TW. Wider patches read and write
// longer contiguous runs per channel plane (better DRAM page locality) at the price of more
// halo rows per output row.
// BN: output channels per workgroup (64 or 128). 64 halves the accumulator registers, so more
// workgroups share a CU and their load / MFMA / store phases overlap.
template <int KH, int KW, int TW = 32, int BN = 64>
struct IgemmGeom {
    static constexpr int TH = IG_PIX / TW;
    static constexpr int HH = TH + KH - 1, WW = TW + KW - 1, TAPS = KH * KW;
    static constexpr int HALO_BYTES = HH * WW * 32;
    static constexpr int W_PITCH = TAPS * 32 + 16;             // odd multiple of 16 B: conflict-free rows
    static constexpr int W_BYTES = BN * W_PITCH;               // one (o tile, channel chunk) slab
    static constexpr int W_PIECES = W_BYTES / 1024;
    static_assert(W_BYTES % 1024 == 0, "slab must be whole 1 KiB wave loads");
    static constexpr int HALO_OFF = (W_BYTES + 1023) / 1024 * 1024;
    static constexpr int LDS_BYTES = HALO_OFF + HALO_BYTES;
    static constexpr int UNITS = HH * WW * 2;                  // (pixel, 8-channel half) staging tasks
    static constexpr int PASSES = (UNITS + 255) / 256;
};

// Where the weight of (input channel c, tap, output channel o) of the convolution a kernel runs lies in w_ref.
// mirror == 0: w_ref is that convolution's own parameter, [(c, tap)][o]. mirror != 0: the kernel runs the data gradient
// of a convolution whose parameter w_ref is ([(c_f, tap_f)][o_f] with C output and O input channels in the kernel's
// terms): its weights are w'[(o_f, tap)][c_f] = w[(c_f, taps - 1 - tap)][o_f], read in place, so that no mirrored
// copy has to be written first.
__device__ __forceinline__ long weight_source_index(int c, int tap, int o, int C, int O, int taps, int mirror) {
    return mirror ? ((long)o * taps + (taps - 1 - tap)) * C + c : ((long)c * taps + tap) * O + o;
}
// The 16 input channels of chunk `chunk` at (tap, output channel o), rounded: h[0] holds channels 0..7, h[1] 8..15
// (zeros past C or O). The pre-passes below give one thread one (row, tap) of a slab, adjacent threads adjacent output
// channels: with a convolution's own parameter each of the 16 reads is contiguous across the wave; with a mirrored one
// the 16 reads of a thread are 64 contiguous bytes (four 16-byte loads when the rows allow it). Either way the thread
// writes its 32 bytes of the image as two 16-byte stores instead of sixteen 2-byte ones.
__device__ __forceinline__ void weight_row_tap(half8_t (&h)[2], const float* __restrict__ w, int chunk, int tap, int o, int C, int O,
                                               int taps, int mirror) {
    const int c0 = chunk * IG_CC;
    if (mirror && o < O && c0 + IG_CC <= C && (C & 3) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0) {
        const floatx4* q = reinterpret_cast<const floatx4*>(w + weight_source_index(c0, tap, o, C, O, taps, 1));
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const floatx4 v = q[i];
#pragma unroll
            for (int j = 0; j < 4; j++) h[i >> 1][(i & 1) * 4 + j] = (_Float16)v[j];
        }
        return;
    }
#pragma unroll
    for (int cc = 0; cc < IG_CC; cc++) {
        const bool ok = c0 + cc < C && o < O;
        const float v = w[ok ? weight_source_index(c0 + cc, tap, o, C, O, taps, mirror) : 0];
        h[cc >> 3][cc & 7] = ok ? (_Float16)v : (_Float16)0.f;
    }
}

// Pre-pass: w_ref [wb][C*TAPS][O] fp32  ->  fp16 slabs [wb][o_tile][chunk][BN][W_PITCH/2].
template <int KH, int KW, int BN>
__global__ __launch_bounds__(256) void conv_weight_image_kernel(_Float16* __restrict__ dst,
                                                                const float* __restrict__ w_ref, int C, int O,
                                                                int n_chunks, int n_otiles, int mirror) {
    using G = IgemmGeom<KH, KW, 32, BN>;
    const int slab = blockIdx.y;                               // (wb * n_otiles + o_tile) * n_chunks + chunk
    const int chunk = slab % n_chunks, o_tile = (slab / n_chunks) % n_otiles, wb = slab / (n_chunks * n_otiles);
    const int t = blockIdx.x * 256 + threadIdx.x;             // (row, tap) within the slab, rows fastest
    const int o_l = t % BN, tap = t / BN;
    if (tap >= G::TAPS) return;
    half8_t h[2];
    weight_row_tap(h, w_ref + (long)wb * C * G::TAPS * O, chunk, tap, o_tile * BN + o_l, C, O, G::TAPS, mirror);
    half8_t* q = reinterpret_cast<half8_t*>(dst + (long)slab * (G::W_BYTES / 2) + o_l * (G::W_PITCH / 2) + tap * IG_CC);
    q[0] = h[0];
    q[1] = h[1];
}

struct IgemmArgs {
    float* y;
    const float* x;
    const _Float16* wimg;
    const float* bias;
    int C, H, W, O, H_out, W_out, pad;
    int n_chunks, n_otiles, tiles_w, tiles_h;
    int w_batched;
    long bias_sp, bias_sc, bias_sn;   // bias element of (image b, pixel, channel o): bias[b*bias_sn + pixel*bias_sp + o*bias_sc]
    int relu;
    int patch_map;                    // resident kernels: 0 strided by the grid, 1 XCD-contiguous, 2 XCD-contiguous runs,
                                      // 3 image-major (per-sample weights: every workgroup stays inside one image);
                                      // 4, 5: 1 and 3 with every XCD on the same eighth of ALL images (a per-pixel bias
                                      // shared by the images is then read once per XCD instead of once per image)
    int n_images;                     // patch_map 3: images of the batch (the grid is a multiple of it wide)
    long w_image_bytes;               // patch_map 3: bytes from one image's weight image to the next
};

// Image b and place r (tile index inside the image) of a patch index. Under patch_map 4 the index runs over (eighth of
// the image, image, place inside the eighth), so that the contiguous range of an XCD is one eighth of every image.
__device__ __forceinline__ void patch_image_and_place(const IgemmArgs& p, int patch, int patches_per_image, int& b, int& r) {
    if (p.patch_map == 4) {
        const int s = patches_per_image >> 3;
        const int blk = patch / s, q = patch - blk * s;
        const int e = blk / p.n_images;
        b = blk - e * p.n_images;
        r = e * s + q;
    } else {
        b = patch / patches_per_image;
        r = patch - b * patches_per_image;
    }
}

// Patches of a workgroup of the resident kernels under patch_map 3, for the reference's Conv2d parameter with one
// weight copy per sample (src/Model.cu:248-252): the grid's G workgroups are split evenly over the images (G / n_images
// each, neighbours in XCD-major order, so that an image's workgroups share an L2 when the counts divide), and a
// workgroup walks its image's patches with that stride. Its weights are those of its image.
__device__ __forceinline__ void image_major_patches(const IgemmArgs& p, int patches_per_image, int& image, int& first_patch,
                                                    int& patch_stride, int& my_patches) {
    const int G = gridDim.x;
    const int wpi = G / p.n_images;
    if (p.patch_map == 5) {
        // (the host checked: G, wpi and patches_per_image are multiples of 8) XCD e holds wpi / 8 workgroups of every
        // image, and they walk the e-th eighth of that image's patches: the eighth of a per-pixel bias that those
        // patches read is the same for all images and stays in the XCD's L2
        const int e = blockIdx.x & 7, slot = blockIdx.x >> 3, wpx = wpi >> 3, s = patches_per_image >> 3;
        image = slot / wpx;
        const int k = slot - image * wpx;
        first_patch = image * patches_per_image + e * s + k;
        patch_stride = wpx;
        my_patches = k < s ? (s - k + wpx - 1) / wpx : 0;
        return;
    }
    const int u = (G % 8 == 0) ? (int)(blockIdx.x & 7) * (G >> 3) + (int)(blockIdx.x >> 3) : (int)blockIdx.x;
    image = u / wpi;
    const int j = u - image * wpi;
    first_patch = image * patches_per_image + j;
    patch_stride = wpi;
    my_patches = j < patches_per_image ? (patches_per_image - j + wpi - 1) / wpi : 0;
}

template <int KH, int KW, int TW, int BN, bool VEC4>
__global__ __launch_bounds__(256, (BN == 64 ? 3 : 2)) void conv_igemm_kernel(const IgemmArgs p) {
    using G = IgemmGeom<KH, KW, TW, BN>;
    constexpr int CB = TW / 32;                                 // 32-pixel MFMA column blocks per patch row
    constexpr int WN = BN / 64, WM = 4 / WN;                    // wave grid: WN over channels, WM over pixel blocks
    constexpr int FP = 8 / WM;                                  // 32-pixel blocks per wave (8 per patch)
    extern __shared__ __attribute__((aligned(1024))) char lds[];
    char* lds_w = lds;
    char* lds_h = lds + G::HALO_OFF;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int li = lane & 31, lh = lane >> 5;
    int tile, o_tile, b;
    xcd_contiguous_block(tile, o_tile, b);
    const int tile_w = tile % p.tiles_w, tile_h = tile / p.tiles_w;
    const int th0 = tile_h * G::TH, tw0 = tile_w * TW;

    const float* xb = p.x + (long)b * p.C * p.H * p.W;
    const char* wsrc = reinterpret_cast<const char*>(p.wimg) +
                       ((long)(p.w_batched ? b : 0) * p.n_otiles + o_tile) * p.n_chunks * G::W_BYTES + lane * 16;

    // Staging tasks of one chunk. "Core" tasks move 4 adjacent pixels x 8 channels: eight 16-byte
    // loads (one per channel plane, whole 128-byte lines per 8 lanes), transposed in registers
    // into four channel-last 16-byte LDS slots. "Edge" tasks move the KW-1 halo columns left and
    // right of the 32-pixel core, one pixel x 8 channels each. VEC4 (W % 4 == 0, aligned x)
    // guarantees a core quad is entirely inside or outside the image.
    constexpr int W4 = TW / 4;                                   // quads per patch row
    constexpr int CORE_TASKS = 2 * G::HH * W4, EDGE_TASKS = 2 * G::HH * (KW - 1);
    static_assert(CORE_TASKS + EDGE_TASKS <= 256, "one task per thread");
    const bool is_core = tid < CORE_TASKS, is_edge = !is_core && tid < CORE_TASKS + EDGE_TASKS;
    int t_h8, t_hh, t_ww;                                        // 8-channel half, halo row, first halo column
    if (is_core) {
        const int w4 = tid % W4;
        t_hh = (tid / W4) % G::HH;
        t_h8 = tid / (W4 * G::HH);
        t_ww = p.pad + 4 * w4;                                   // halo column of image column tw0 + 4*w4
    } else {
        const int e = tid - CORE_TASKS;
        const int ecol = (KW > 1) ? e % (KW - 1) : 0;
        t_hh = (KW > 1) ? (e / (KW - 1)) % G::HH : 0;
        t_h8 = (KW > 1) ? e / ((KW - 1) * G::HH) : 0;
        t_ww = ecol < p.pad ? ecol : TW + ecol;
    }
    const int t_hin = th0 + t_hh - p.pad, t_win = tw0 + t_ww - p.pad;
    const bool row_ok = (is_core || is_edge) && t_hin >= 0 && t_hin < p.H;
    bool col_ok[4];
#pragma unroll
    for (int q = 0; q < 4; q++) col_ok[q] = row_ok && t_win + q >= 0 && t_win + q < p.W && (is_core || q == 0);
    const int t_off = row_ok ? t_hin * p.W + (t_win < 0 ? 0 : (t_win >= p.W ? p.W - 1 : t_win)) : 0;
    const bool quad_ok = VEC4 && col_ok[0];                      // whole quad in range, 16-byte aligned

    floatx16 acc[2][FP];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < FP; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    const long plane = (long)p.H * p.W;
    floatx4 raw[8];                                              // [channel][pixel of the quad]

    auto load_halo = [&](int chunk) {
        const int c0 = chunk * IG_CC + t_h8 * 8;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const bool c_ok = c0 + e < p.C;
            const float* src = xb + (c_ok ? (long)(c0 + e) * plane : 0) + t_off;
            floatx4 v = {0.f, 0.f, 0.f, 0.f};
            if (VEC4) {
                if (is_core) {
                    const floatx4 q = *reinterpret_cast<const floatx4*>(quad_ok ? src : xb);
                    v = (quad_ok && c_ok) ? q : v;
                } else {
                    const float q = *src;
                    v[0] = (col_ok[0] && c_ok) ? q : 0.f;
                }
            } else {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const float f = *(col_ok[q] ? src + q : xb);
                    v[q] = (col_ok[q] && c_ok) ? f : 0.f;
                }
            }
            raw[e] = v;
        }
    };
    auto store_halo = [&]() {
        if (!(is_core || is_edge)) return;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            if (q > 0 && !is_core) break;
            half8_t h;
#pragma unroll
            for (int e = 0; e < 8; e++) h[e] = (_Float16)raw[e][q];
            const int ww = t_ww + q;
            *reinterpret_cast<half8_t*>(lds_h + (t_hh * G::WW + ww) * 32 + ((t_h8 ^ ((ww >> 3) & 1)) << 4)) = h;
        }
    };
    auto load_slab = [&](int chunk) {
        for (int j = wave; j < G::W_PIECES; j += 4)
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void*)(wsrc + (long)chunk * G::W_BYTES + j * 1024),
                (__attribute__((address_space(3))) void*)(lds_w + j * 1024), 16, 0, 0);
    };

    load_halo(0);
    load_slab(0);
    // The sums start from the bias, so the epilogue is stores only (a load issued after stores is not counted as
    // returned before those stores are acknowledged: bias loads between the blocks of stores made every block wait for
    // the one before). Per channel: one load per channel and workgroup, handed out through LDS; per pixel: read where
    // the results will go, lanes on adjacent pixels.
    if (p.bias) {
        const bool o_full = o_tile * BN + BN <= p.O;
        if (p.bias_sp == 0) {
            float* lds_b = reinterpret_cast<float*>(lds_h);      // the halo area is free until the first store_halo
            if (tid < BN) {
                const int o = o_tile * BN + tid;
                lds_b[tid] = o < p.O ? p.bias[(long)b * p.bias_sn + (long)o * p.bias_sc] : 0.f;
            }
            __syncthreads();
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const floatx4 v = *reinterpret_cast<const floatx4*>(lds_b + wn * 64 + i * 32 + g * 8 + lh * 4);
#pragma unroll
                    for (int j = 0; j < FP; j++)
#pragma unroll
                        for (int e = 0; e < 4; e++) acc[i][j][g * 4 + e] = v[e];
                }
            __syncthreads();                                    // read before the first halo lands in the same bytes
        } else {
#pragma unroll
            for (int j = 0; j < FP; j++) {
                const int blk = wm * FP + j;
                const int ho = th0 + blk / CB, wo = tw0 + (blk % CB) * 32 + li;
                const bool px_ok = ho < p.H_out && wo < p.W_out;
                const float* bp = p.bias + (long)b * p.bias_sn + (px_ok ? ((long)ho * p.W_out + wo) * p.bias_sp : 0);
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int o = o_tile * BN + wn * 64 + lh * 4 + i * 32 + (r >> 2) * 8 + (r & 3);
                        const bool ok = px_ok && (o_full || o < p.O);
                        const float v = bp[(long)(ok ? o : 0) * p.bias_sc];
                        acc[i][j][r] = ok ? v : 0.f;
                    }
            }
        }
    }
    for (int chunk = 0; chunk < p.n_chunks; chunk++) {
        store_halo();                                           // registers (chunk) -> LDS, fp16 channel-last
        __builtin_amdgcn_s_waitcnt(0x0070 | 0x0F00);            // vmcnt(0): this wave's slab pieces landed
        __syncthreads();
        if (chunk + 1 < p.n_chunks) load_halo(chunk + 1);       // lands while the MFMAs below run
#pragma unroll
        for (int kh = 0; kh < KH; kh++) {
#pragma unroll
            for (int kw = 0; kw < KW; kw++) {
                const int tap = kh * KW + kw;
                half8_t wf[2], pf[FP];
#pragma unroll
                for (int i = 0; i < 2; i++)
                    wf[i] = *reinterpret_cast<const half8_t*>(lds_w + (wn * 64 + i * 32 + li) * G::W_PITCH + tap * 32 + lh * 16);
#pragma unroll
                for (int j = 0; j < FP; j++) {
                    const int blk = wm * FP + j;                  // pixel block: patch row blk / CB, column block blk % CB
                    const int col = (blk % CB) * 32 + li + kw;
                    pf[j] = *reinterpret_cast<const half8_t*>(lds_h + ((blk / CB + kh) * G::WW + col) * 32 +
                                                               ((lh ^ ((col >> 3) & 1)) << 4));
                }
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int j = 0; j < FP; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[i], pf[j], acc[i][j], 0, 0, 0);
            }
        }
        __syncthreads();                                        // everyone is done reading this chunk's LDS
        if (chunk + 1 < p.n_chunks) load_slab(chunk + 1);
    }

    // ---- epilogue: activation + NCHW store (lanes = adjacent pixels) --------------------------
    float* yb = p.y + (long)b * p.O * p.H_out * p.W_out;
    const long hw_out = (long)p.H_out * p.W_out;
    const int o_base = o_tile * BN + wn * 64 + lh * 4;
    const bool o_full = o_tile * BN + BN <= p.O;
#pragma unroll
    for (int j = 0; j < FP; j++) {
        const int blk = wm * FP + j;
        const int ho = th0 + blk / CB, wo = tw0 + (blk % CB) * 32 + li;
        if (ho >= p.H_out || wo >= p.W_out) continue;
        const long pix = (long)ho * p.W_out + wo;
        float* dst = yb + pix;
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int o = o_base + i * 32 + (r >> 2) * 8 + (r & 3);
                float v = acc[i][j][r];
                if (p.relu) v = v > 0.f ? v : 0.f;
                if (o_full || o < p.O) dst[(long)o * hw_out] = v;
            }
    }
}

// ---- implicit GEMM with the whole weight set resident in LDS -------------------------------
// When O <= 128 per tile and C*KH*KW*128 fp16 weights (plus one halo) fit in the 160 KiB of LDS,
// a persistent workgroup loads the weights ONCE and then walks over pixel patches. This removes
// the per-patch weight re-fetch (half of the L1 fill traffic of the streaming-slab kernel) and
// lets the epilogue stores of one patch drain while the next patch is staged and computed.
// Weight rows are unpadded (TAPS*32 bytes); rows o and o+8 would share LDS banks, so the two
// 16-byte halves of every (row, tap) are swapped when bit 3 of the row is set.
template <int KH, int KW, int BN>
__global__ __launch_bounds__(256) void conv_weight_image_resident_kernel(_Float16* __restrict__ dst,
                                                                         const float* __restrict__ w_ref, int C,
                                                                         int O, int n_chunks, int n_otiles, int mirror) {
    constexpr int TAPS = KH * KW;
    // blockIdx.z: weight copy (one per sample for the reference's Conv2d parameter); images follow each other
    w_ref += (long)blockIdx.z * C * TAPS * O;
    dst += (long)blockIdx.z * n_otiles * n_chunks * (BN * TAPS * IG_CC);
    const int slab = blockIdx.y;                               // o_tile * n_chunks + chunk
    const int chunk = slab % n_chunks, o_tile = slab / n_chunks;
    const int t = blockIdx.x * 256 + threadIdx.x;             // (row, tap) within the slab, rows fastest
    const int o_l = t % BN, tap = t / BN;
    if (tap >= TAPS) return;
    half8_t h[2];
    weight_row_tap(h, w_ref, chunk, tap, o_tile * BN + o_l, C, O, TAPS, mirror);
    half8_t* q = reinterpret_cast<half8_t*>(dst + (long)slab * (BN * TAPS * IG_CC) + o_l * (TAPS * IG_CC) + tap * IG_CC);
    const int swap = (o_l >> 3) & 1;
    q[swap] = h[0];
    q[swap ^ 1] = h[1];
}

// PIX_BIAS: the bias varies per pixel (the reference's Bias node after the matmul); otherwise it is
// absent or per channel and is fetched once per workgroup.
//
// Eight waves, two per SIMD. Wave (wm, wn) owns 64 pixels (two 32-pixel blocks) x 64 channels of
// the 256 x 128 patch tile. A work item is one 16-channel chunk of one patch:
//     store_halo (registers -> fp16 LDS)  | barrier |  MFMAs, with the loads of the halo two items
//     ahead issued one behind every other filter tap  | barrier
// A wave held up at the memory pipe leaves the matrix pipe to its partner on the SIMD. After the
// last chunk of a patch every wave writes its 64 x 64 results (bias already in the accumulator,
// activation on the way out).
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));

// NI: 32-channel blocks per wave; the channel tile of a workgroup is BN = 64 * NI (128 or 64) output channels.
template <int KH, int KW, int TW, bool VEC4, bool PIX_BIAS, int NI>
__global__ __launch_bounds__(512) void conv_igemm_resident_kernel(const IgemmArgs p, const int n_patches) {
    using G = IgemmGeom<KH, KW, TW, 128>;
    constexpr int BN = 64 * NI, WCH = 32 * NI, CB = TW / 32, FP = 2, NW = 8;   // WCH: channels per wave
    constexpr int W_PITCH = G::TAPS * 32, W_CHUNK = BN * W_PITCH;           // unpadded rows
    static_assert(W_CHUNK % 1024 == 0, "chunk must be whole 1 KiB wave loads");
    extern __shared__ __attribute__((aligned(1024))) char lds[];
    char* lds_w = lds;
    char* lds_h = lds + p.n_chunks * W_CHUNK;
    float* lds_bias = reinterpret_cast<float*>(lds_h + G::HALO_BYTES);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int li = lane & 31, lh = lane >> 5;
    const int o_tile = blockIdx.y;
    const int patches_per_image = p.tiles_w * p.tiles_h;
    const long plane = (long)p.H * p.W;

    int w_image = 0, first_patch = blockIdx.x, patch_stride = gridDim.x;
    int my_patches = (n_patches - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;
    if (p.patch_map == 3 || p.patch_map == 5) image_major_patches(p, patches_per_image, w_image, first_patch, patch_stride, my_patches);

    // resident weights: n_chunks * W_CHUNK bytes, 1 KiB per wave-wide request
    {
        const char* wsrc = reinterpret_cast<const char*>(p.wimg) + (long)w_image * p.w_image_bytes +
                           (long)o_tile * p.n_chunks * W_CHUNK + lane * 16;
        const int pieces = p.n_chunks * (W_CHUNK / 1024);
        for (int j = wave; j < pieces; j += NW)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(wsrc + (long)j * 1024),
                                             (__attribute__((address_space(3))) void*)(lds_w + j * 1024), 16, 0, 0);
    }
    float my_bias = 0.f;                                         // requested now, parked in LDS before the first patch
    if (!PIX_BIAS && p.bias && tid < BN && o_tile * BN + tid < p.O) my_bias = p.bias[(long)(o_tile * BN + tid) * p.bias_sc];

    // Staging task of this thread: 4 adjacent pixels x 4 channels ("core": four 16-byte loads, one
    // per channel plane, transposed in registers into four channel-last 8-byte LDS slots) or one
    // halo-column pixel x 4 channels ("edge").
    constexpr int W4 = TW / 4;
    constexpr int CORE_TASKS = 4 * G::HH * W4, EDGE_TASKS = 4 * G::HH * (KW - 1);
    static_assert(CORE_TASKS + EDGE_TASKS <= 512, "one task per thread");
    const bool is_core = tid < CORE_TASKS, is_edge = !is_core && tid < CORE_TASKS + EDGE_TASKS;
    int t_q4, t_hh, t_ww;                                        // channel quarter, halo row, first halo column
    if (is_core) {
        t_hh = (tid / W4) % G::HH;
        t_q4 = tid / (W4 * G::HH);
        t_ww = p.pad + 4 * (tid % W4);
    } else {
        const int e = tid - CORE_TASKS;
        const int ecol = (KW > 1) ? e % (KW > 1 ? KW - 1 : 1) : 0;
        t_hh = (KW > 1) ? (e / (KW > 1 ? KW - 1 : 1)) % G::HH : 0;
        t_q4 = (KW > 1) ? e / ((KW > 1 ? KW - 1 : 1) * G::HH) : 0;
        t_ww = ecol < p.pad ? ecol : TW + ecol;
    }
    t_q4 &= 3;
    auto halo_slot = [&](int hh, int ww) {                       // 8-byte slot of this thread's channel quarter
        return lds_h + (hh * G::WW + ww) * 32 + (((t_q4 >> 1) ^ ((ww >> 3) & 1)) << 4) + (t_q4 & 1) * 8;
    };

    // Patches of this workgroup: first_patch + pi * patch_stride, pi < my_patches. Workgroups go to the
    // eight XCDs round-robin by their linear index and every XCD has an L2 of its own, so (when the grid
    // is a multiple of 8 wide) the workgroups of one XCD share a contiguous eighth of the patches: halo
    // rows and columns that neighbouring patches have in common are then found in that L2 instead of
    // being fetched again from memory.
    if (p.patch_map != 0 && p.patch_map != 3 && p.patch_map != 5 && gridDim.x % 8 == 0) {
        const int xcd = blockIdx.x & 7, q = blockIdx.x >> 3, nq = gridDim.x >> 3;
        const int lo = (int)((long)n_patches * xcd / 8), hi = (int)((long)n_patches * (xcd + 1) / 8);
        if (p.patch_map == 1 || p.patch_map == 4) {              // the XCD's workgroups sweep its range side by side
            first_patch = lo + q;
            patch_stride = nq;
            my_patches = q < hi - lo ? (hi - lo - q + nq - 1) / nq : 0;
        } else {                                                 // every workgroup walks a run of its own
            const int a = lo + (int)((long)(hi - lo) * q / nq), b = lo + (int)((long)(hi - lo) * (q + 1) / nq);
            first_patch = a;
            patch_stride = 1;
            my_patches = b - a;
        }
    }
    // work items of this workgroup: (patch, chunk) pairs
    // Items per patch are rounded up to an even count: an odd chunk count gets one empty item
    // (zero halo, no MFMAs) so that every patch starts on the same register set.
    const int n_items = (p.n_chunks + 1) & ~1;
    const int total = my_patches * n_items;

    // Staging is split in "request" (load_item, two items ahead) and "consume" (store_halo).
    // Requests are unconditional loads from clamped, always valid addresses; padding pixels and
    // channels past C are zeroed at consumption through nv[] (number of valid channels of the
    // thread's 4, 0 for a pixel outside the image). With VEC4 an edge pixel is fetched as the
    // aligned quad that holds it (component t_comp), so every lane issues the same instruction.
    floatx4 raw[2][4];
    int nv[2] = {0, 0};
    const int t_comp = (t_ww - p.pad) & 3;
    int ld_patch = first_patch, ld_chunk = 0, ld_it = 0;
    const float* ld_src = p.x;                                   // this thread's pixel, channel t_q4*4, current patch
    bool ld_ok = false;                                          // the pixel (VEC4: its quad) is inside the image
    int ld_hin = 0, ld_win = 0;
    // A request is issued in three steps so that its four loads can be spread between the MFMAs of
    // the item in progress: load_begin (addresses), load_one x 4, load_end (advance to the next item).
    // Past the last item the requests are still issued (to the first quad of x, results unused):
    // a fixed number of requests per item lets every wait name exactly the set it needs.
    const float* ld_cur = p.x;
    int ld_n = 0, ld_c0 = 0;
    auto load_begin = [&](int& nvalid) {
        if (ld_chunk == 0) {                                     // new patch: redo the geometry (uniform branch)
            const bool live = ld_it < total;
            const int patch = live ? ld_patch : 0;
            int b, r;
            patch_image_and_place(p, patch, patches_per_image, b, r);
            const int th0 = (r / p.tiles_w) * G::TH, tw0 = (r % p.tiles_w) * TW;
            ld_hin = th0 + t_hh - p.pad;
            ld_win = tw0 + t_ww - p.pad;
            const bool row_ok = live && (is_core || is_edge) && ld_hin >= 0 && ld_hin < p.H;
            ld_ok = row_ok && (!VEC4 || (ld_win >= 0 && ld_win < p.W));   // W % 4 == 0: a quad is all in or all out
            ld_src = p.x + ((long)b * p.C + t_q4 * 4) * plane +
                     (ld_ok ? (long)ld_hin * p.W + (VEC4 ? (ld_win & ~3) : ld_win) : 0);
        }
        ld_c0 = ld_chunk * IG_CC + t_q4 * 4;
        int n = p.C - ld_c0;
        n = n < 0 ? 0 : (n > 4 ? 4 : n);
        ld_n = ld_ok ? n : 0;
        nvalid = VEC4 ? ld_n : 4;
        // lanes without work read the first quad of x; channels past n repeat the last valid one
        ld_cur = ld_n > 0 ? ld_src + (long)ld_chunk * IG_CC * plane : p.x;
    };
    auto load_one = [&](floatx4 (&dst)[4], const int e) {
        if (VEC4) {
            dst[e] = *reinterpret_cast<const floatx4*>(ld_cur);
            ld_cur += plane & -(long)(e + 1 < ld_n);
        } else {
            floatx4 v = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const bool ok = e < ld_n && ld_win + q >= 0 && ld_win + q < p.W && (is_core || q == 0);
                const float f = *(ok ? ld_cur + (long)e * plane + q : p.x);
                v[q] = ok ? f : 0.f;
            }
            dst[e] = v;
        }
    };
    auto load_end = [&]() {
        ld_it++;
        if (++ld_chunk == n_items) { ld_chunk = 0; ld_patch += patch_stride; }
    };
    auto load_item = [&](floatx4 (&dst)[4], int& nvalid) {
        load_begin(nvalid);
#pragma unroll
        for (int e = 0; e < 4; e++) load_one(dst, e);
        load_end();
    };
    auto store_halo = [&](const floatx4 (&src)[4], const int nvalid) {
        // Every lane takes delivery of the set here, also lanes without a task: a request left
        // pending on some path would force a full drain before the registers are reused.
#pragma unroll
        for (int e = 0; e < 4; e++) asm volatile("" ::"v"(src[e]));
        if (!(is_core || is_edge)) return;
        if (is_core) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                half4_t h;
#pragma unroll
                for (int e = 0; e < 4; e++) h[e] = e < nvalid ? (_Float16)src[e][q] : (_Float16)0.f;
                *reinterpret_cast<half4_t*>(halo_slot(t_hh, t_ww + q)) = h;
            }
        } else {
            half4_t h;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                float f = src[e][0];
                if (VEC4) {
                    f = t_comp == 1 ? src[e][1] : f;
                    f = t_comp == 2 ? src[e][2] : f;
                    f = t_comp == 3 ? src[e][3] : f;
                }
                h[e] = e < nvalid ? (_Float16)f : (_Float16)0.f;
            }
            *reinterpret_cast<half4_t*>(halo_slot(t_hh, t_ww)) = h;
        }
    };

    // A per-channel bias (or zero) is the starting value of every accumulator; the 128 values of the
    // channel tile sit in LDS behind the halo and are read back at the start of each patch.
    floatx16 acc[NI][FP];
    auto init_acc = [&]() {
#pragma unroll
        for (int i = 0; i < NI; i++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const floatx4 bq = *reinterpret_cast<const floatx4*>(lds_bias + wn * WCH + i * 32 + g * 8 + lh * 4);
#pragma unroll
                for (int j = 0; j < FP; j++)
#pragma unroll
                    for (int q = 0; q < 4; q++) acc[i][j][g * 4 + q] = bq[q];
            }
    };

    // Two fragment sets: the LDS reads of tap t + 1 are issued before the MFMAs of tap t, so the
    // matrix pipe does not wait for LDS latency at every tap.
    // after_tap(tap) runs behind the MFMAs of each tap (used to spread the next halo request). It
    // sits outside the branch on `live`, so an empty item (odd chunk count) issues the same requests
    // as a full one without touching LDS or the matrix pipe.
    auto compute = [&](int chunk, const bool live, auto after_tap) {
        const char* wbase = lds_w + chunk * W_CHUNK + (wn * WCH + li) * W_PITCH + ((lh ^ ((li >> 3) & 1)) << 4);
        half8_t wf[2][NI], pf[2][FP];
        auto read_frags = [&](const int tap, half8_t (&w)[NI], half8_t (&x)[FP]) {
            const int kh = tap / KW, kw = tap % KW;
#pragma unroll
            for (int i = 0; i < NI; i++)
                w[i] = *reinterpret_cast<const half8_t*>(wbase + i * 32 * W_PITCH + tap * 32);
#pragma unroll
            for (int j = 0; j < FP; j++) {
                const int blk = wm * FP + j;
                const int col = (blk % CB) * 32 + li + kw;
                x[j] = *reinterpret_cast<const half8_t*>(lds_h + ((blk / CB + kh) * G::WW + col) * 32 +
                                                          ((lh ^ ((col >> 3) & 1)) << 4));
            }
        };
        if (live) read_frags(0, wf[0], pf[0]);
#pragma unroll
        for (int tap = 0; tap < G::TAPS; tap++) {
            if (live) {
                if (tap + 1 < G::TAPS) read_frags(tap + 1, wf[(tap + 1) & 1], pf[(tap + 1) & 1]);
                __builtin_amdgcn_sched_barrier(0);               // requests stay ahead of the MFMAs below
#pragma unroll
                for (int i = 0; i < NI; i++)
#pragma unroll
                    for (int j = 0; j < FP; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[tap & 1][i], pf[tap & 1][j], acc[i][j], 0, 0, 0);
            }
            after_tap(tap);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    const int o_wave = o_tile * BN + wn * WCH;                   // uniform; lane channel = o_wave + lh*4 + i*32 + ...
    const bool o_full = o_tile * BN + BN <= p.O;                 // uniform: whole channel tile exists
    const long hw_out = (long)p.H_out * p.W_out;

    // Write unit (j, i) of the finished patch: pixel block j x 32 channels, 16 stores per lane.
    // bias (if per pixel) + activation + NCHW store, lanes = adjacent pixels. The address of a store
    // is a wave-uniform channel plane (scalar registers, stepped with scalar adds) plus one per-lane
    // byte offset shared by the 16 stores: pixel, and 4 planes up for the upper half-wave.
    // A patch that lies wholly inside the output takes the unpredicated path.
    // The per-pixel bias of unit (j, i), requested one unit ahead of its use (the first unit's at the start of the
    // patch): a request issued after a unit's stores would not be counted as returned before those stores are.
    auto bias_request = [&](float (&bv)[16], const int j, const int i, const int patch) {
        int b, r;
            patch_image_and_place(p, patch, patches_per_image, b, r);
        const int th0 = (r / p.tiles_w) * G::TH, tw0 = (r % p.tiles_w) * TW;
        const int blk = wm * FP + j;
        const int ho = th0 + blk / CB, wo = tw0 + (blk % CB) * 32 + li;
        const long pix = (ho < p.H_out && wo < p.W_out) ? (long)ho * p.W_out + wo : 0;
        const int o_lane = o_wave + i * 32 + lh * 4;
        const float* bp = p.bias + (long)b * p.bias_sn + pix * p.bias_sp;
#pragma unroll
        for (int rr = 0; rr < 16; rr++) {
            const int o = o_lane + (rr >> 2) * 8 + (rr & 3);
            bv[rr] = bp[(long)((o_full || o < p.O) ? o : 0) * p.bias_sc];
        }
    };
    auto flush_unit = [&](const int j, const int i, const int patch, const float (&bv)[16]) {
        int b, r;
            patch_image_and_place(p, patch, patches_per_image, b, r);
        const int th0 = (r / p.tiles_w) * G::TH, tw0 = (r % p.tiles_w) * TW;
        const int blk = wm * FP + j;
        const int ho = th0 + blk / CB, wo = tw0 + (blk % CB) * 32 + li;
        const bool inside = o_full && th0 + G::TH <= p.H_out && tw0 + TW <= p.W_out;   // uniform
        const bool pix_ok = inside || (ho < p.H_out && wo < p.W_out);
        const long pix = pix_ok ? (long)ho * p.W_out + wo : 0;
        const unsigned lane_bytes = (unsigned)((pix + (long)lh * 4 * hw_out) * 4);
        char* pl = reinterpret_cast<char*>(p.y + ((long)b * p.O + o_wave + i * 32) * hw_out);
        const int o_lane = o_wave + i * 32 + lh * 4;
        auto finished = [&](const int rr) {
            float v = acc[i][j][rr];
            if (PIX_BIAS) v += bv[rr];                           // a per-channel bias is already in the accumulator
            return fmaxf(v, p.relu ? 0.f : v);                  // NaN -> 0 under ReLU, like x > 0 ? x : 0
        };
        // The step between channel planes is opaque so that the plane addresses are not precomputed
        // and kept in registers across the whole kernel.
        int step_lo = __builtin_amdgcn_readfirstlane((int)(hw_out * 4)),
            step_hi = __builtin_amdgcn_readfirstlane((int)((hw_out * 4) >> 32));
        asm volatile("" : "+s"(step_lo), "+s"(step_hi));
        const long step1 = ((long)step_hi << 32) | (unsigned)step_lo, step5 = step1 * 5;
        if (inside) {
#pragma unroll
            for (int rr = 0; rr < 16; rr++) {
                *reinterpret_cast<float*>(pl + lane_bytes) = finished(rr);
                pl += (rr & 3) == 3 ? step5 : step1;             // channels +1 +1 +1 +5: 0..3, 8..11, 16..19, 24..27
            }
        } else {
#pragma unroll
            for (int rr = 0; rr < 16; rr++) {
                const int o = o_lane + (rr >> 2) * 8 + (rr & 3);
                const float v = finished(rr);
                if (pix_ok && o < p.O) *reinterpret_cast<float*>(pl + lane_bytes) = v;
                pl += (rr & 3) == 3 ? step5 : step1;
            }
        }
    };

    // LDS-only barrier: waits for this wave's LDS traffic, not for the global requests in flight.
    auto lds_barrier = []() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
    // One work item. The register set r (parity of the item index) is a compile-time choice, so
    // nothing is copied and a set's requests stay in flight across a whole item.
    auto item = [&](floatx4 (&r)[4], int& n, const int c) {
        store_halo(r, n);                                        // registers -> LDS (waits for this set only)
        lds_barrier();
        // Request the item two ahead into the same set: one load behind every other tap, so a wave
        // held up at the memory pipe leaves the matrix pipe to its partner on the SIMD.
        load_begin(n);
        compute(c, c < p.n_chunks, [&](const int tap) {
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (tap == (2 * e + 1 < G::TAPS ? 2 * e + 1 : G::TAPS - 1)) load_one(r, e);
        });
        load_end();
        lds_barrier();                                           // halo may be overwritten
    };

    load_item(raw[0], nv[0]);
    load_item(raw[1], nv[1]);
    if (tid < BN) lds_bias[tid] = my_bias;
    __builtin_amdgcn_s_waitcnt(0x0070 | 0x0F00);                 // vmcnt(0): resident weights landed
    lds_barrier();
    float bvs[2][16];
    for (int pi = 0; pi < my_patches; pi++) {
        init_acc();
        const int patch = first_patch + pi * patch_stride;
        if (PIX_BIAS) bias_request(bvs[0], 0, 0, patch);         // lands under the patch's MFMAs
        for (int c = 0; c < n_items; c += 2) {
            item(raw[0], nv[0], c);
            item(raw[1], nv[1], c + 1);
        }
#pragma unroll
        for (int j = 0; j < FP; j++)
#pragma unroll
            for (int i = 0; i < NI; i++) {
                constexpr int UNITS = FP * NI;
                const int u = j * NI + i;
                if (PIX_BIAS && u + 1 < UNITS) bias_request(bvs[(u + 1) & 1], (u + 1) / NI, (u + 1) % NI, patch);
                flush_unit(j, i, patch, bvs[u & 1]);
            }
    }
}

// ---- resident weights, two halo buffers (3x3, 64-pixel-wide patches, 16-byte image rows) --------------
// The kernel above spends a quarter of every work item between its two barriers: the halo is stored, the
// workgroup meets, multiplies, meets again. With a second halo buffer the next item's halo is stored in the
// middle of the current item's MFMAs and one barrier per item is left. LDS has no room for it beside nine
// taps of weights (144 KiB for 128 channels x 64 x 9), so the ninth tap is not resident: a wave requests the
// 16 bytes per lane and 32 output channels it needs of it one item ahead, from L2, into registers. The other
// eight taps make rows of exactly 256 bytes; their sixteen 16-byte slots (tap, channel half) are stored at
// slot ^ (row & 15), so the sixteen rows of a read pass fall on sixteen different bank groups.
// Image of one channel tile: [chunk][BN rows][256 B] for taps 0..7, then [chunk][BN rows][32 B] for tap 8.
template <int BN>
__global__ __launch_bounds__(256) void conv_weight_image_db_kernel(_Float16* __restrict__ dst, const float* __restrict__ w_ref,
                                                                   int C, int O, int n_chunks, int n_otiles, int mirror) {
    // One thread per (row, tap) of a slab: 16 reads that are contiguous across the threads of a wave (adjacent
    // output channels; with mirrored weights the 16 reads of a thread are the contiguous ones) and two 16-byte
    // stores, instead of one 2-byte store per element.
    // blockIdx.z: weight copy (one per sample for the reference's Conv2d parameter); images follow each other
    w_ref += (long)blockIdx.z * C * 9 * O;
    dst += (long)blockIdx.z * n_otiles * n_chunks * BN * 144;
    const int slab = blockIdx.y;                               // o_tile * n_chunks + chunk
    const int chunk = slab % n_chunks, o_tile = slab / n_chunks;
    const int t = blockIdx.x * 256 + threadIdx.x;
    const int o_l = t % BN, tap = t / BN;
    if (tap >= 9) return;
    const int o = o_tile * BN + o_l;
    half8_t h[2];
    weight_row_tap(h, w_ref, chunk, tap, o, C, O, 9, mirror);
    _Float16* tile = dst + (long)o_tile * n_chunks * BN * 144;   // 288 bytes per (chunk, row)
#pragma unroll
    for (int half = 0; half < 2; half++) {
        _Float16* q = tap < 8 ? tile + ((long)chunk * BN + o_l) * 128 + (((tap * 2 + half) ^ (o_l & 15)) << 3)
                              : tile + (long)n_chunks * BN * 128 + ((long)chunk * BN + o_l) * 16 + half * 8;
        *reinterpret_cast<half8_t*>(q) = h[half];
    }
}

// NCH: channel chunks of 16 (= ceil(C / 16), even, so that an item's parity is its chunk's). Work item k (one chunk of one patch) multiplies out of halo buffer k & 1; behind its
// first four taps it requests item k + 2 into the register set item k's halo came from, behind its sixth tap
// it rounds item k + 1's set into the other halo buffer, and it ends with the only barrier.
constexpr int CONV_DB_PLANE = 6 * 66 * 16 + 96;               // halo plane pitch of the kernel below: 6432 = 25 * 256 + 32
template <bool PIX_BIAS, int NI, int NCH>
__global__ __launch_bounds__(512) void conv3x3_resident_db_kernel(const IgemmArgs p, const int n_patches) {
    using G = IgemmGeom<3, 3, 64, 128>;
    constexpr int TW = 64, KW = 3;
    constexpr int BN = 64 * NI, WCH = 32 * NI, CB = TW / 32, FP = 2, NW = 8;
    constexpr int W_CHUNK = BN * 256;
    static_assert(NCH % 2 == 0, "items come in pairs");
    // A halo buffer is two planes (channels 0..7 and 8..15 of the chunk), 16 bytes per pixel. Fragment reads
    // (32 adjacent pixels of one plane per half-wave) and the staging stores below are then conflict-free
    // without a swizzle; the plane pitch is 32 bytes past a multiple of 256 so that the two planes a 16-lane
    // group of stores touches use different banks.
    constexpr int H_PLANE = CONV_DB_PLANE, H_BYTES = 2 * H_PLANE;
    static_assert(H_PLANE >= G::HH * G::WW * 16 && H_PLANE % 256 == 32, "plane pitch");
    extern __shared__ __attribute__((aligned(1024))) char lds[];
    char* lds_w = lds;
    char* lds_h0 = lds + NCH * W_CHUNK;
    char* lds_h1 = lds_h0 + H_BYTES;
    float* lds_bias = reinterpret_cast<float*>(lds_h1 + H_BYTES);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int li = lane & 31, lh = lane >> 5;
    const int o_tile = blockIdx.y;
    const int patches_per_image = p.tiles_w * p.tiles_h;
    const long plane = (long)p.H * p.W;

    int w_image = 0, first_patch = blockIdx.x, patch_stride = gridDim.x;
    int my_patches = (n_patches - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;
    if (p.patch_map == 3 || p.patch_map == 5) image_major_patches(p, patches_per_image, w_image, first_patch, patch_stride, my_patches);

    const char* wtile = reinterpret_cast<const char*>(p.wimg) + (long)w_image * p.w_image_bytes + (long)o_tile * NCH * BN * 288;
    {
        const char* wsrc = wtile + lane * 16;
        constexpr int pieces = NCH * (W_CHUNK / 1024);
        for (int j = wave; j < pieces; j += NW)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(wsrc + (long)j * 1024),
                                             (__attribute__((address_space(3))) void*)(lds_w + j * 1024), 16, 0, 0);
    }
    // tap 8 of this wave's channels: the set of the chunk in hand and the set of the next chunk, requested one
    // item ahead from the image (it stays in L2: every workgroup reads the same 16 KiB)
    half8_t w8[2][NI];
    const char* w8_src = wtile + (long)NCH * W_CHUNK + ((wn * WCH + li) * 32 + lh * 16);
    auto request_w8 = [&](half8_t (&dst)[NI], const int c) {
#pragma unroll
        for (int i = 0; i < NI; i++) dst[i] = *reinterpret_cast<const half8_t*>(w8_src + (c * BN + i * 32) * 32);
    };
    request_w8(w8[0], 0);
    float my_bias = 0.f;
    if (!PIX_BIAS && p.bias && tid < BN && o_tile * BN + tid < p.O) my_bias = p.bias[(long)(o_tile * BN + tid) * p.bias_sc];

    // staging task of this thread: 4 adjacent pixels x 4 channels (core) or one halo-column pixel x 4 channels
    // (edge). A wave takes one halo row; its lanes are (channel quarter, pixel quad) with the quarter fastest, so
    // the 16 lanes of a store pass write the four quarters of four quads: 16 different 8-byte bank pairs.
    constexpr int W4 = TW / 4;
    constexpr int CORE_TASKS = 4 * G::HH * W4, EDGE_TASKS = 4 * G::HH * (KW - 1);
    static_assert(CORE_TASKS + EDGE_TASKS <= 512 && W4 == 16, "one task per thread, one halo row per wave");
    const bool is_core = tid < CORE_TASKS, is_edge = !is_core && tid < CORE_TASKS + EDGE_TASKS;
    int t_q4, t_hh, t_ww;
    if (is_core) {
        t_q4 = tid & 3;
        t_hh = tid >> 6;
        t_ww = p.pad + 4 * ((tid >> 2) & 15);
    } else {
        const int e = tid - CORE_TASKS;
        const int ecol = e % (KW - 1);
        t_hh = (e / (KW - 1)) % G::HH;
        t_q4 = e / ((KW - 1) * G::HH);
        t_ww = ecol < p.pad ? ecol : TW + ecol;
    }
    t_q4 &= 3;
    auto halo_slot = [&](char* hb, int hh, int ww) {
        return hb + (t_q4 >> 1) * H_PLANE + (hh * G::WW + ww) * 16 + (t_q4 & 1) * 8;
    };

    if (p.patch_map != 0 && p.patch_map != 3 && p.patch_map != 5 && gridDim.x % 8 == 0) {   // the workgroups of an XCD sweep a contiguous eighth
        const int xcd = blockIdx.x & 7, q = blockIdx.x >> 3, nq = gridDim.x >> 3;
        const int lo = (int)((long)n_patches * xcd / 8), hi = (int)((long)n_patches * (xcd + 1) / 8);
        first_patch = lo + q;
        patch_stride = nq;
        my_patches = q < hi - lo ? (hi - lo - q + nq - 1) / nq : 0;
    }
    const int total = my_patches * NCH;

    // requests: unconditional loads from clamped addresses, zeroed at consumption through nv[]
    floatx4 raw[2][4];
    int nv[2] = {0, 0};
    const int t_comp = (t_ww - p.pad) & 3;
    int ld_patch = first_patch, ld_chunk = 0, ld_it = 0;
    const float* ld_src = p.x;
    bool ld_ok = false;
    int ld_hin = 0, ld_win = 0;
    const float* ld_cur = p.x;
    int ld_n = 0, ld_c0 = 0;
    auto load_begin = [&](int& nvalid) {
        if (ld_chunk == 0) {
            const bool live = ld_it < total;
            const int patch = live ? ld_patch : 0;
            int b, r;
            patch_image_and_place(p, patch, patches_per_image, b, r);
            const int th0 = (r / p.tiles_w) * G::TH, tw0 = (r % p.tiles_w) * TW;
            ld_hin = th0 + t_hh - p.pad;
            ld_win = tw0 + t_ww - p.pad;
            const bool row_ok = live && (is_core || is_edge) && ld_hin >= 0 && ld_hin < p.H;
            ld_ok = row_ok && ld_win >= 0 && ld_win < p.W;       // W % 4 == 0: a quad is all in or all out
            ld_src = p.x + ((long)b * p.C + t_q4 * 4) * plane + (ld_ok ? (long)ld_hin * p.W + (ld_win & ~3) : 0);
        }
        ld_c0 = ld_chunk * IG_CC + t_q4 * 4;
        int n = p.C - ld_c0;
        n = n < 0 ? 0 : (n > 4 ? 4 : n);
        ld_n = ld_ok ? n : 0;
        nvalid = ld_n;
        ld_cur = ld_n > 0 ? ld_src + (long)ld_chunk * IG_CC * plane : p.x;
    };
    auto load_one = [&](floatx4 (&dst)[4], const int e) {
        dst[e] = *reinterpret_cast<const floatx4*>(ld_cur);
        ld_cur += plane & -(long)(e + 1 < ld_n);
    };
    auto load_end = [&]() {
        ld_it++;
        if (++ld_chunk == NCH) { ld_chunk = 0; ld_patch += patch_stride; }
    };
    auto load_item = [&](floatx4 (&dst)[4], int& nvalid) {
        load_begin(nvalid);
#pragma unroll
        for (int e = 0; e < 4; e++) load_one(dst, e);
        load_end();
    };
    auto store_halo = [&](const floatx4 (&src)[4], const int nvalid, char* hb) {
#pragma unroll
        for (int e = 0; e < 4; e++) asm volatile("" ::"v"(src[e]));   // every lane takes delivery of the set
        if (!(is_core || is_edge)) return;
        if (is_core) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                half4_t h;
#pragma unroll
                for (int e = 0; e < 4; e++) h[e] = e < nvalid ? (_Float16)src[e][q] : (_Float16)0.f;
                *reinterpret_cast<half4_t*>(halo_slot(hb, t_hh, t_ww + q)) = h;
            }
        } else {
            half4_t h;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                float f = src[e][0];
                f = t_comp == 1 ? src[e][1] : f;
                f = t_comp == 2 ? src[e][2] : f;
                f = t_comp == 3 ? src[e][3] : f;
                h[e] = e < nvalid ? (_Float16)f : (_Float16)0.f;
            }
            *reinterpret_cast<half4_t*>(halo_slot(hb, t_hh, t_ww)) = h;
        }
    };

    floatx16 acc[NI][FP];
    auto init_acc = [&]() {
#pragma unroll
        for (int i = 0; i < NI; i++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const floatx4 bq = *reinterpret_cast<const floatx4*>(lds_bias + wn * WCH + i * 32 + g * 8 + lh * 4);
#pragma unroll
                for (int j = 0; j < FP; j++)
#pragma unroll
                    for (int q = 0; q < 4; q++) acc[i][j][g * 4 + q] = bq[q];
            }
    };

    // chunk c out of halo buffer hb, ninth tap out of w9; after_tap(tap) runs behind the MFMAs of each tap
    auto compute = [&](const int c, const char* hb, const half8_t (&w9)[NI], auto after_tap) {
        const char* wrow = lds_w + c * W_CHUNK + (wn * WCH + li) * 256;
        const int sw = li & 15;
        half8_t wf[2][NI], pf[2][FP];
        auto read_frags = [&](const int tap, half8_t (&w)[NI], half8_t (&x)[FP]) {
            const int kh = tap / KW, kw = tap % KW;
#pragma unroll
            for (int i = 0; i < NI; i++)
                w[i] = tap < 8 ? *reinterpret_cast<const half8_t*>(wrow + i * 32 * 256 + (((tap * 2 + lh) ^ sw) << 4)) : w9[i];
#pragma unroll
            for (int j = 0; j < FP; j++) {
                const int blk = wm * FP + j;
                const int col = (blk % CB) * 32 + li + kw;
                x[j] = *reinterpret_cast<const half8_t*>(hb + lh * H_PLANE + ((blk / CB + kh) * G::WW + col) * 16);
            }
        };
        read_frags(0, wf[0], pf[0]);
#pragma unroll
        for (int tap = 0; tap < 9; tap++) {
            if (tap + 1 < 9) read_frags(tap + 1, wf[(tap + 1) & 1], pf[(tap + 1) & 1]);
            __builtin_amdgcn_sched_barrier(0);                   // requests stay ahead of the MFMAs below
#pragma unroll
            for (int i = 0; i < NI; i++)
#pragma unroll
                for (int j = 0; j < FP; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[tap & 1][i], pf[tap & 1][j], acc[i][j], 0, 0, 0);
            after_tap(tap);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    const int o_wave = o_tile * BN + wn * WCH;
    const bool o_full = o_tile * BN + BN <= p.O;
    const long hw_out = (long)p.H_out * p.W_out;
    // The per-pixel bias of unit (j, i), requested one unit ahead of its use (the first unit's at the start of the
    // patch): a request issued after a unit's stores would not be counted as returned before those stores are.
    auto bias_request = [&](float (&bv)[16], const int j, const int i, const int patch) {
        int b, r;
            patch_image_and_place(p, patch, patches_per_image, b, r);
        const int th0 = (r / p.tiles_w) * G::TH, tw0 = (r % p.tiles_w) * TW;
        const int blk = wm * FP + j;
        const int ho = th0 + blk / CB, wo = tw0 + (blk % CB) * 32 + li;
        const long pix = (ho < p.H_out && wo < p.W_out) ? (long)ho * p.W_out + wo : 0;
        const int o_lane = o_wave + i * 32 + lh * 4;
        const float* bp = p.bias + (long)b * p.bias_sn + pix * p.bias_sp;
#pragma unroll
        for (int rr = 0; rr < 16; rr++) {
            const int o = o_lane + (rr >> 2) * 8 + (rr & 3);
            bv[rr] = bp[(long)((o_full || o < p.O) ? o : 0) * p.bias_sc];
        }
    };
    auto flush_unit = [&](const int j, const int i, const int patch, const float (&bv)[16]) {
        int b, r;
            patch_image_and_place(p, patch, patches_per_image, b, r);
        const int th0 = (r / p.tiles_w) * G::TH, tw0 = (r % p.tiles_w) * TW;
        const int blk = wm * FP + j;
        const int ho = th0 + blk / CB, wo = tw0 + (blk % CB) * 32 + li;
        const bool inside = o_full && th0 + G::TH <= p.H_out && tw0 + TW <= p.W_out;   // uniform
        const bool pix_ok = inside || (ho < p.H_out && wo < p.W_out);
        const long pix = pix_ok ? (long)ho * p.W_out + wo : 0;
        const unsigned lane_bytes = (unsigned)((pix + (long)lh * 4 * hw_out) * 4);
        char* pl = reinterpret_cast<char*>(p.y + ((long)b * p.O + o_wave + i * 32) * hw_out);
        const int o_lane = o_wave + i * 32 + lh * 4;
        auto finished = [&](const int rr) {
            float v = acc[i][j][rr];
            if (PIX_BIAS) v += bv[rr];
            return fmaxf(v, p.relu ? 0.f : v);                  // NaN -> 0 under ReLU, like x > 0 ? x : 0
        };
        int step_lo = __builtin_amdgcn_readfirstlane((int)(hw_out * 4)),
            step_hi = __builtin_amdgcn_readfirstlane((int)((hw_out * 4) >> 32));
        asm volatile("" : "+s"(step_lo), "+s"(step_hi));        // plane addresses are stepped, not kept in registers
        const long step1 = ((long)step_hi << 32) | (unsigned)step_lo, step5 = step1 * 5;
        if (inside) {
#pragma unroll
            for (int rr = 0; rr < 16; rr++) {
                *reinterpret_cast<float*>(pl + lane_bytes) = finished(rr);
                pl += (rr & 3) == 3 ? step5 : step1;
            }
        } else {
#pragma unroll
            for (int rr = 0; rr < 16; rr++) {
                const int o = o_lane + (rr >> 2) * 8 + (rr & 3);
                const float v = finished(rr);
                if (pix_ok && o < p.O) *reinterpret_cast<float*>(pl + lane_bytes) = v;
                pl += (rr & 3) == 3 ? step5 : step1;
            }
        }
    };

    auto lds_barrier = []() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
    // Item k multiplies out of halo buffer k & 1. Register set (k + 1) & 1 holds item k + 1, requested two items
    // ago: behind tap 4 (waves 0..3) or tap 6 (waves 4..7: the two waves of a SIMD, w and w + 4, do not round at
    // the same time) it is rounded into the other halo buffer, and the set is at once requested again for item
    // k + 3, one load behind each of the following taps. One barrier ends the item.
    auto item = [&](floatx4 (&nxt)[4], int& n_nxt, const int c, const char* hb_cur, char* hb_next, const half8_t (&w9)[NI],
                    half8_t (&w9_next)[NI]) {
        compute(c, hb_cur, w9, [&](const int tap) {
            if (tap == 3) request_w8(w9_next, c + 1 < NCH ? c + 1 : 0);
            if (wave < 4) {
                if (tap == 4) {
                    store_halo(nxt, n_nxt, hb_next);
                    load_begin(n_nxt);
                }
                if (tap >= 5) load_one(nxt, tap - 5);
            } else {
                if (tap == 6) {
                    store_halo(nxt, n_nxt, hb_next);
                    load_begin(n_nxt);
                    load_one(nxt, 0);
                    load_one(nxt, 1);
                }
                if (tap == 7) load_one(nxt, 2);
                if (tap == 8) load_one(nxt, 3);
            }
        });
        load_end();
        lds_barrier();                                           // next halo complete, this one free again
    };

    load_item(raw[0], nv[0]);
    load_item(raw[1], nv[1]);
    if (tid < BN) lds_bias[tid] = my_bias;
    __builtin_amdgcn_s_waitcnt(0x0070 | 0x0F00);                 // vmcnt(0): resident weights and both sets landed
    store_halo(raw[0], nv[0], lds_h0);
    load_item(raw[0], nv[0]);                                    // item 2
    lds_barrier();
    float bvs[2][16];
    for (int pi = 0; pi < my_patches; pi++) {
        init_acc();
        const int patch = first_patch + pi * patch_stride;
        if (PIX_BIAS) bias_request(bvs[0], 0, 0, patch);         // lands under the patch's MFMAs
#pragma unroll 1
        for (int c = 0; c < NCH; c += 2) {
            item(raw[1], nv[1], c, lds_h0, lds_h1, w8[0], w8[1]);
            item(raw[0], nv[0], c + 1, lds_h1, lds_h0, w8[1], w8[0]);
        }
#pragma unroll
        for (int j = 0; j < FP; j++)
#pragma unroll
            for (int i = 0; i < NI; i++) {
                constexpr int UNITS = FP * NI;
                const int u = j * NI + i;
                if (PIX_BIAS && u + 1 < UNITS) bias_request(bvs[(u + 1) & 1], (u + 1) / NI, (u + 1) % NI, patch);
                flush_unit(j, i, patch, bvs[u & 1]);
            }
    }
    // the requests issued for items past the end are still in flight
    __builtin_amdgcn_s_waitcnt(0x0070 | 0x0F00);
}

static bool conv_igemm_applicable(size_t C, size_t O, size_t K_h, size_t K_w, size_t stride, size_t pad, size_t N) {
    (void)O;
    // pad <= K_w - 1 keeps the 32 aligned core columns of a tile inside its halo
    return stride == 1 && ((K_h == 3 && K_w == 3) || (K_h == 1 && K_w == 1)) && pad <= K_w - 1 && C >= 8 && N <= 65535;
}

// Per-sample weights (one copy per image) on the resident kernels: the grid must split evenly over the images, at
// least one workgroup each. Returns the grid width (0: not possible, the per-patch slab kernel takes the layer).
static int resident_grid_per_sample(size_t N, int n_otiles) {
    const int per_tile = device_cu_count() / n_otiles;
    if (N == 0 || N > (size_t)per_tile) return 0;
    return (int)(per_tile / (int)N * (int)N);
}

// A per-pixel bias that all images share (the reference's Bias node after the product, src/Model.cu:252-256) is read by
// every patch of every image: 16 x 64 x 128 x 128 -> 128 reads its 8 MB sixteen times. With every XCD on the same eighth
// of all images, that eighth stays in the XCD's L2 (patch maps 4 and 5 in place of 1 and 3; the grid, the workgroups
// per image and the patches per image have to be multiples of 8).
static int resident_patch_map(int map, const float* bias, int64_t bias_sp, int64_t bias_sn, int grid_x, size_t N, size_t patches_per_image) {
    static const char* env = getenv("NZHIP_CONV_BIAS_MAP");          // benchmarking only: 0 keeps maps 1 and 3
    if (env && atoi(env) == 0) return map;
    if (!bias || bias_sp == 0 || bias_sn != 0 || N < 2 || grid_x % 8 != 0 || patches_per_image % 8 != 0) return map;
    if (map == 1) return 4;
    if (map == 3 && grid_x % (int)N == 0 && (grid_x / (int)N) % 8 == 0) return 5;
    return map;
}

// Key of a weight image: everything the conversion kernel's output depends on (image kind, tile shape, source and extents).
static void conv_image_key(uint64_t (&key)[PREPARED_KEY_WORDS], int kind, int kh, int kw, int bn, const float* w_ref, size_t C,
                           size_t O, int n_chunks, int n_otiles, size_t w_batch, bool w_mirror) {
    for (auto& k : key) k = 0;
    key[0] = (uint64_t)kind | ((uint64_t)kh << 8) | ((uint64_t)kw << 16) | ((uint64_t)bn << 24) | ((uint64_t)(w_mirror ? 1 : 0) << 40);
    key[1] = reinterpret_cast<uintptr_t>(w_ref);
    key[2] = C; key[3] = O; key[4] = (uint64_t)n_chunks; key[5] = (uint64_t)n_otiles; key[6] = w_batch;
}

template <int KH, int KW, int TW, int BN>
static int conv_igemm_launch(float* y, const float* x, const float* w_ref, const float* bias, size_t N, size_t C,
                             size_t H, size_t W, size_t O, size_t pad, size_t w_batch, int64_t bias_sp,
                             int64_t bias_sc, int64_t bias_sn, int act, size_t H_out, size_t W_out, bool w_mirror, hipStream_t s) {
    using G = IgemmGeom<KH, KW, TW, BN>;
    const int n_chunks = (int)((C + IG_CC - 1) / IG_CC), n_otiles = (int)((O + BN - 1) / BN);
    if (n_otiles > 65535) return set_error(NZHIP_E_UNSUPPORTED, "nzhip_conv2d_forward: too many output channels");
    // Resident weights with two halo buffers: 3x3, 64-wide patches, 16-byte image rows, and one of the chunk counts
    // the kernel is built for (2 or 4 chunks of 16 input channels with a 128-channel tile; 2, 4 or 8 with a 64-channel
    // tile, whose eight chunks still fit LDS).
    if constexpr (KH == 3 && KW == 3 && TW == 64) {
        constexpr int NI = BN / 64;
        static const char* db_env = getenv("NZHIP_CONV_DB");     // 0: the single-buffer kernel (benchmarking only)
        const bool vec4r = (W % 4 == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0);
        const bool pixb = bias && bias_sp != 0;                  // per-pixel bias with a 128-channel tile: out of registers
        const bool count_ok = n_chunks == 2 || n_chunks == 4 || (n_chunks == 8 && NI == 1);
        const int grid_ps = w_batch > 1 ? resident_grid_per_sample(N, n_otiles) : 0;
        if (!(db_env && atoi(db_env) == 0) && (w_batch == 1 || grid_ps > 0) && count_ok && vec4r && !(pixb && NI == 2)) {
            auto run = [&](auto nch_tag) -> int {
                constexpr int NCH = decltype(nch_tag)::value;
                constexpr size_t lds_need = (size_t)NCH * BN * 256 + 4 * CONV_DB_PLANE + 128 * sizeof(float);
                static_assert(lds_need <= 160 * 1024 - 512, "LDS budget");
                const size_t image_bytes = (size_t)n_otiles * NCH * BN * 288, bytes = image_bytes * w_batch;
                uint64_t key[PREPARED_KEY_WORDS];
                conv_image_key(key, 1, 3, 3, BN, w_ref, C, O, NCH, n_otiles, w_batch, w_mirror);
                ImageLease lease;
                if (int rc = image_acquire(PREPARED_CONV_W, key, bytes, s, &lease)) return rc;
                _Float16* wres = static_cast<_Float16*>(lease.ptr);
                dim3 pg((unsigned)((BN * 9 + 255) / 256), (unsigned)(n_otiles * NCH), (unsigned)w_batch);
                if (lease.fill)
                    hipLaunchKernelGGL((conv_weight_image_db_kernel<BN>), pg, dim3(256), 0, s, wres, w_ref, (int)C, (int)O, NCH, n_otiles, w_mirror ? 1 : 0);
                IgemmArgs a;
                a.y = y; a.x = x; a.wimg = wres; a.bias = bias;
                a.C = (int)C; a.H = (int)H; a.W = (int)W; a.O = (int)O; a.H_out = (int)H_out; a.W_out = (int)W_out;
                a.pad = (int)pad; a.n_chunks = NCH; a.n_otiles = n_otiles;
                a.tiles_w = (int)((W_out + TW - 1) / TW);
                a.tiles_h = (int)((H_out + G::TH - 1) / G::TH);
                a.w_batched = 0; a.bias_sp = bias_sp; a.bias_sc = bias_sc; a.bias_sn = bias_sn; a.relu = act == NZHIP_ACT_RELU;
                a.patch_map = w_batch > 1 ? 3 : 1;
                a.n_images = (int)N; a.w_image_bytes = (long)image_bytes;
                const long n_patches = (long)N * a.tiles_w * a.tiles_h;
                int rc = NZHIP_OK;
                if (n_patches > 0x7fffffffL) rc = set_error(NZHIP_E_UNSUPPORTED, "nzhip_conv2d_forward: too many patches");
                auto kdb = conv3x3_resident_db_kernel<false, NI, NCH>;
                if constexpr (NI == 1) {
                    if (pixb) kdb = conv3x3_resident_db_kernel<true, NI, NCH>;
                }
                if (rc == NZHIP_OK)
                    rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kdb), (int)lds_need, "hipFuncSetAttribute(conv3x3_resident_db)");
                if (rc == NZHIP_OK) {
                    const int cus = device_cu_count();
                    int per_tile = cus / n_otiles > 0 ? cus / n_otiles : 1;      // one workgroup per CU in total
                    if ((long)per_tile > n_patches) per_tile = (int)n_patches;
                    if (w_batch > 1) per_tile = grid_ps;                          // a whole number of workgroups per image
                    a.patch_map = resident_patch_map(a.patch_map, bias, bias_sp, bias_sn, per_tile, N, (size_t)a.tiles_w * a.tiles_h);
                    hipLaunchKernelGGL(kdb, dim3((unsigned)per_tile, (unsigned)n_otiles, 1), dim3(512), lds_need, s, a, (int)n_patches);
                    hipError_t e = hipGetLastError();
                    if (e != hipSuccess) rc = set_hip_error(e, "conv3x3_resident_db kernel launch");
                }
                int rc2 = image_release(lease, s, rc == NZHIP_OK);
                return rc ? rc : rc2;
            };
            if (n_chunks == 2) return run(std::integral_constant<int, 2>{});
            if (n_chunks == 4) return run(std::integral_constant<int, 4>{});
            if constexpr (NI == 1) return run(std::integral_constant<int, 8>{});
        }
    }
    // Resident-weight route: shared weights whose fp16 image (unpadded) plus one halo fit in LDS.
    {
        constexpr size_t W_CHUNK_R = BN * (size_t)G::TAPS * 32;
        constexpr int NI = BN / 64;
        const size_t lds_need = (size_t)n_chunks * W_CHUNK_R + G::HALO_BYTES + 128 * sizeof(float);   // + bias
        static const char* res_env = getenv("NZHIP_CONV_RESIDENT");
        const bool allow = res_env ? atoi(res_env) != 0 : true;
        const int grid_ps = w_batch > 1 ? resident_grid_per_sample(N, n_otiles) : 0;
        if (allow && (w_batch == 1 || grid_ps > 0) && lds_need <= 160 * 1024 - 512) {
            const size_t image_bytes = (size_t)n_otiles * n_chunks * W_CHUNK_R, bytes = image_bytes * w_batch;
            uint64_t key[PREPARED_KEY_WORDS];
            conv_image_key(key, 2, KH, KW, BN, w_ref, C, O, n_chunks, n_otiles, w_batch, w_mirror);
            ImageLease lease;
            if (int rc = image_acquire(PREPARED_CONV_W, key, bytes, s, &lease)) return rc;
            _Float16* wres = static_cast<_Float16*>(lease.ptr);
            dim3 pg((unsigned)((BN * G::TAPS + 255) / 256), (unsigned)(n_otiles * n_chunks), (unsigned)w_batch);
            if (lease.fill)
                hipLaunchKernelGGL((conv_weight_image_resident_kernel<KH, KW, BN>), pg, dim3(256), 0, s, wres, w_ref, (int)C,
                                   (int)O, n_chunks, n_otiles, w_mirror ? 1 : 0);
            IgemmArgs a;
            a.y = y; a.x = x; a.wimg = wres; a.bias = bias;
            a.C = (int)C; a.H = (int)H; a.W = (int)W; a.O = (int)O; a.H_out = (int)H_out; a.W_out = (int)W_out;
            a.pad = (int)pad; a.n_chunks = n_chunks; a.n_otiles = n_otiles;
            a.tiles_w = (int)((W_out + TW - 1) / TW);
            a.tiles_h = (int)((H_out + G::TH - 1) / G::TH);
            a.w_batched = 0; a.bias_sp = bias_sp; a.bias_sc = bias_sc; a.bias_sn = bias_sn; a.relu = act == NZHIP_ACT_RELU;
            static const char* map_env = getenv("NZHIP_CONV_PATCH_MAP");
            a.patch_map = w_batch > 1 ? 3 : (map_env ? atoi(map_env) : 1);
            a.n_images = (int)N; a.w_image_bytes = (long)image_bytes;
            const long n_patches = (long)N * a.tiles_w * a.tiles_h;
            int rc = NZHIP_OK;
            if (n_patches > 0x7fffffffL) rc = set_error(NZHIP_E_UNSUPPORTED, "nzhip_conv2d_forward: too many patches");
            const bool vec4r = (W % 4 == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0);
            const bool pixb = bias && bias_sp != 0;
            auto kres = vec4r ? (pixb ? conv_igemm_resident_kernel<KH, KW, TW, true, true, NI>
                                      : conv_igemm_resident_kernel<KH, KW, TW, true, false, NI>)
                              : (pixb ? conv_igemm_resident_kernel<KH, KW, TW, false, true, NI>
                                      : conv_igemm_resident_kernel<KH, KW, TW, false, false, NI>);
            if (rc == NZHIP_OK)
                rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kres), (int)lds_need, "hipFuncSetAttribute(conv_igemm_resident)");
            if (rc == NZHIP_OK) {
                const int cus = device_cu_count();
                int per_tile = cus / n_otiles > 0 ? cus / n_otiles : 1;      // one workgroup per CU in total
                if ((long)per_tile > n_patches) per_tile = (int)n_patches;
                if (w_batch > 1) per_tile = grid_ps;                          // a whole number of workgroups per image
                a.patch_map = resident_patch_map(a.patch_map, bias, bias_sp, bias_sn, per_tile, N, (size_t)a.tiles_w * a.tiles_h);
                dim3 grid((unsigned)per_tile, (unsigned)n_otiles, 1);
                hipLaunchKernelGGL(kres, grid, dim3(512), lds_need, s, a, (int)n_patches);
                hipError_t e = hipGetLastError();
                if (e != hipSuccess) rc = set_hip_error(e, "conv_igemm_resident kernel launch");
            }
            int rc2 = image_release(lease, s, rc == NZHIP_OK);
            return rc ? rc : rc2;
        }
    }
    const size_t slabs = (size_t)w_batch * n_otiles * n_chunks;
    if (slabs > 65535) return set_error(NZHIP_E_UNSUPPORTED, "nzhip_conv2d_forward: weight set too large for the fused route");
    uint64_t key[PREPARED_KEY_WORDS];
    conv_image_key(key, 3, KH, KW, BN, w_ref, C, O, n_chunks, n_otiles, w_batch, w_mirror);
    ImageLease lease;
    if (int rc = image_acquire(PREPARED_CONV_W, key, slabs * G::W_BYTES, s, &lease)) return rc;
    _Float16* wimg = static_cast<_Float16*>(lease.ptr);
    int rc = NZHIP_OK;
    if (lease.fill) {
        // pad bytes of the slabs are never read as data; no need to clear them
        dim3 grid((unsigned)((BN * G::TAPS + 255) / 256), (unsigned)slabs);
        hipLaunchKernelGGL((conv_weight_image_kernel<KH, KW, BN>), grid, dim3(256), 0, s, wimg, w_ref, (int)C, (int)O,
                           n_chunks, n_otiles, w_mirror ? 1 : 0);
    }
    if (rc == NZHIP_OK) {
        IgemmArgs a;
        a.y = y;
        a.x = x;
        a.wimg = wimg;
        a.bias = bias;
        a.C = (int)C;
        a.H = (int)H;
        a.W = (int)W;
        a.O = (int)O;
        a.H_out = (int)H_out;
        a.W_out = (int)W_out;
        a.pad = (int)pad;
        a.n_chunks = n_chunks;
        a.n_otiles = n_otiles;
        a.tiles_w = (int)((W_out + TW - 1) / TW);
        a.tiles_h = (int)((H_out + G::TH - 1) / G::TH);
        a.w_batched = w_batch > 1;
        a.bias_sp = bias_sp;
        a.bias_sc = bias_sc;
        a.bias_sn = bias_sn;
        a.relu = act == NZHIP_ACT_RELU;
        a.patch_map = 0;
        a.n_images = (int)N; a.w_image_bytes = 0;
        const bool vec4 = (W % 4 == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0);
        auto kfn = vec4 ? conv_igemm_kernel<KH, KW, TW, BN, true> : conv_igemm_kernel<KH, KW, TW, BN, false>;
        if (rc == NZHIP_OK)
            rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kfn), G::LDS_BYTES, "hipFuncSetAttribute(conv_igemm)");
        if (rc == NZHIP_OK) {
            dim3 grid((unsigned)(a.tiles_w * a.tiles_h), (unsigned)n_otiles, (unsigned)N);
            hipLaunchKernelGGL(kfn, grid, dim3(256), G::LDS_BYTES, s, a);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) rc = set_hip_error(e, "conv_igemm kernel launch");
        }
    }
    int rc2 = image_release(lease, s, rc == NZHIP_OK);
    return rc ? rc : rc2;
}

// ---- implicit GEMM for any kernel extent and stride ----------------------------------------------------------
// The kernels above are built for 3x3 and 1x1 at stride 1 (halo geometry and tap loops are compile-time). Every other
// geometry whose rows allow 16-byte loads -- 5x5, strides 2..4, rectangular kernels -- used to write its column matrix
// (K_h K_w times the input) and read it back through the GEMM. This kernel keeps the same arithmetic without it:
// a workgroup of eight waves owns a segment of 256 output pixels (256 / SW output rows x SW columns, SW the power of
// two >= 16 that covers the output width) x BN output channels of one image. Per chunk of 16 input channels it
// stages the input rows under the segment in LDS as fp16, channel-last (32 bytes per pixel, the two 16-byte halves
// swapped every eight columns like the fixed-geometry kernels), and the chunk's weight slab (BN rows of taps x 32
// bytes + 16, direct to LDS); a tap's B fragment is then one 16-byte read per lane at (row * stride + r,
// column * stride + s). A thread's staging tasks -- four adjacent input columns x eight channels, transposed in
// registers -- are fixed for the whole kernel; the next chunk's loads are in flight while this one multiplies.
constexpr int CG_PX = 256, CG_THREADS = 512, CG_TP_MAX = 3;

struct ConvGenArgs {
    float* y;
    const float* x;
    const _Float16* wimg;   // [w copy][o tile][chunk][BN][w_pitch / 2]
    const float* bias;
    int C, H, W, O, Ho, Wo, Kh, Kw, stride, pad;
    int n_chunks, n_otiles, w_batched;
    int sw_log, span, pw, shift, segs_w;
    int w_pitch, slab_bytes, halo_off;
    long bias_sp, bias_sc, bias_sn;
    int relu;
    int img_chunks, halo_plane;           // chunks per channel tile in the weight image (n_chunks rounded up to CPB); bytes of one halo plane
    int bias_map;                         // a per-pixel bias shared by the images: every XCD on one stretch of segments of ALL images
    int chunk_groups, chunks_per_group;   // the contraction split over groups of channel chunks (blockIdx.z = image * groups + group)
    float* partial;                       // with more than one group: [group][image][O][Ho * Wo] sums without bias or activation
};

// Pre-pass: w_ref [wb][C * taps][O] fp32 -> fp16 slabs [wb][o tile][chunk][BN][taps * 16 + 8]
__global__ __launch_bounds__(256) void conv_weight_image_gen_kernel(_Float16* __restrict__ dst, const float* __restrict__ w_ref, int C,
                                                                    int O, int taps, int BN, int w_pitch_halfs, int n_chunks,
                                                                    int n_otiles, int mirror) {
    const int slab = blockIdx.y;                               // (wb * n_otiles + o_tile) * n_chunks + chunk
    const int chunk = slab % n_chunks, o_tile = (slab / n_chunks) % n_otiles, wb = slab / (n_chunks * n_otiles);
    const int t = blockIdx.x * 256 + threadIdx.x;             // (row, tap) within the slab, rows fastest
    const int o_l = t % BN, tap = t / BN;
    if (tap >= taps) return;
    half8_t h[2];
    weight_row_tap(h, w_ref + (long)wb * C * taps * O, chunk, tap, o_tile * BN + o_l, C, O, taps, mirror);
    half8_t* q = reinterpret_cast<half8_t*>(dst + (long)slab * BN * w_pitch_halfs + (long)o_l * w_pitch_halfs + tap * IG_CC);
    q[0] = h[0];
    q[1] = h[1];
}

// NO: 32-channel blocks per wave (BN / 64); every wave also owns two 32-pixel blocks. TP: staging tasks per thread.
// VEC: image rows are whole 16-byte pieces (W a multiple of 4, aligned x): a task's four columns are one load per
// channel and lie inside or outside the image together; otherwise (14 x 14 images ...) four loads with their own bounds.
// PIXB: the bias varies per pixel (the reference's Bias node after the matmul; the per-image bias of an in-place data gradient).
// CPB: 16-channel chunks per loop step (p.n_chunks counts steps). With 2, a step stages two halo planes and two slabs and
// multiplies 2 x taps times between its two barriers: the store / barrier / request phases, which cost as much as the 9
// taps of a 3x3 chunk, are paid half as often (layers with many channels; 16 x 256 x 56 x 56 -> 256: 124 -> 95 us).
template <int NO, int TP, bool VEC, bool PIXB, int CPB>
__global__ __launch_bounds__(CG_THREADS) void conv_igemm_gen_kernel(const ConvGenArgs p) {
    constexpr int BN = NO * 64;
    extern __shared__ __attribute__((aligned(1024))) char lds[];
    char* lds_w = lds;
    char* lds_h = lds + p.halo_off;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lh = lane >> 5;
    const int wm = wave & 3, wn = wave >> 2;                    // pixel blocks 2 wm, 2 wm + 1; channel blocks NO wn ..
    // neighbouring segments share input rows: the compute units of one XCD take a contiguous run of them
    int seg_x, o_tile, bz;
    if (PIXB && p.bias_sn == 0 && p.bias_map) xcd_contiguous_block_z_fastest(seg_x, o_tile, bz);   // a bias all images share
    else xcd_contiguous_block(seg_x, o_tile, bz);
    const int b = bz / p.chunk_groups, group = bz % p.chunk_groups;
    const int chunk_lo = group * p.chunks_per_group;
    const int chunk_hi = chunk_lo + p.chunks_per_group < p.n_chunks ? chunk_lo + p.chunks_per_group : p.n_chunks;
    const int SW = 1 << p.sw_log, SR = CG_PX >> p.sw_log;
    const int ho0 = (seg_x / p.segs_w) * SR, wo0 = (seg_x % p.segs_w) * SW;
    const int hb = ho0 * p.stride - p.pad, wf = wo0 * p.stride - p.pad - p.shift;   // image position of staged (0, 0)
    const int taps = p.Kh * p.Kw;
    const long plane = (long)p.H * p.W;
    const float* xb = p.x + (long)b * p.C * plane;
    const char* wsrc = reinterpret_cast<const char*>(p.wimg) +
                       ((long)(p.w_batched ? b : 0) * p.n_otiles + o_tile) * p.img_chunks * p.slab_bytes + lane * 16;

    // staging tasks: task e = tid + 512 k is (8-channel group of the step's 16 CPB channels, staged row, column quad)
    const int pw4 = p.pw >> 2, n_tasks = 2 * CPB * p.span * pw4;
    int t_off[TP], t_dst[TP];                                   // image offset of the quad's first column, LDS byte offset of its first pixel (or -1)
    int t_h8[TP];                                               // bits 0..3: which of the four columns are inside the image; bits 4..: the 8-channel group
#pragma unroll
    for (int k = 0; k < TP; k++) {
        const int e = tid + CG_THREADS * k;
        const int q = e % pw4, row = (e / pw4) % p.span, h8 = e / (pw4 * p.span);
        const int h = hb + row, w = wf + 4 * q;
        const bool row_in = e < n_tasks && h >= 0 && h < p.H;
        int mask = 0;
#pragma unroll
        for (int j = 0; j < 4; j++) mask |= (row_in && w + j >= 0 && w + j < p.W) ? 1 << j : 0;     // VEC: all four or none
        t_off[k] = h * p.W + w;
        t_dst[k] = e < n_tasks ? (row * p.pw + 4 * q) * 32 : -1;
        t_h8[k] = mask | (h8 << 4);
    }

    floatx16 acc[NO][2];
#pragma unroll
    for (int i = 0; i < NO; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    floatx4 raw[TP][8];                                          // [task][channel][pixel of the quad]
    auto load_halo = [&](const int chunk) {
#pragma unroll
        for (int k = 0; k < TP; k++) {
            const int c0 = chunk * (IG_CC * CPB) + (t_h8[k] >> 4) * 8;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const bool c_ok = c0 + e < p.C;
                if (VEC) {
                    const bool ok = (t_h8[k] & 1) && c_ok;
                    raw[k][e] = *reinterpret_cast<const floatx4*>(xb + (ok ? (long)(c0 + e) * plane + t_off[k] : 0));
                } else {
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const bool ok = (t_h8[k] >> j & 1) && c_ok;
                        raw[k][e][j] = xb[ok ? (long)(c0 + e) * plane + t_off[k] + j : 0];
                    }
                }
            }
        }
    };
    auto store_halo = [&](const int chunk) {
#pragma unroll
        for (int k = 0; k < TP; k++) {
            if (t_dst[k] < 0) continue;
            const int g8 = t_h8[k] >> 4, h8 = g8 & 1;            // 8-channel group of the step; half of its 16-channel plane
            const int c0 = chunk * (IG_CC * CPB) + g8 * 8;
            const int col0 = (t_dst[k] >> 5) % p.pw;            // staged column of the quad's first pixel (a multiple of 4)
            char* plane_h = lds_h + (CPB > 1 ? (g8 >> 1) * p.halo_plane : 0);
#pragma unroll
            for (int q = 0; q < 4; q++) {
                half8_t h;
#pragma unroll
                for (int e = 0; e < 8; e++) h[e] = ((t_h8[k] >> q & 1) && c0 + e < p.C) ? (_Float16)raw[k][e][q] : (_Float16)0.f;
                const int col = col0 + q;
                *reinterpret_cast<half8_t*>(plane_h + t_dst[k] + q * 32 + ((h8 ^ ((col >> 3) & 1)) << 4)) = h;
            }
        }
    };
    auto load_slab = [&](const int chunk) {
        const int pieces = (CPB * p.slab_bytes) >> 10;          // the step's slabs follow each other in the image
        for (int j = wave; j < pieces; j += CG_THREADS / 64)
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void*)(wsrc + (long)chunk * (CPB * p.slab_bytes) + j * 1024),
                (__attribute__((address_space(3))) void*)(lds_w + j * 1024), 16, 0, 0);
    };

    // this lane's two pixels: staged row and column of tap (0, 0)
    int prow[2], pcol[2];
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int px = (wm * 2 + j) * 32 + li;
        prow[j] = (px >> p.sw_log) * p.stride;
        pcol[j] = (px & (SW - 1)) * p.stride + p.shift;
    }
    const char* wrow[NO];
#pragma unroll
    for (int i = 0; i < NO; i++) wrow[i] = lds_w + ((wn * NO + i) * 32 + li) * p.w_pitch + lh * 16;

    load_halo(chunk_lo);
    load_slab(chunk_lo);
    // Bias. Loads between the epilogue's blocks of stores would each wait until the stores before them are
    // acknowledged (a load issued after stores is not counted as returned before they are), and every lane asking
    // memory for its own per-channel values sends thousands of requests per workgroup to the same few lines. So a
    // per-channel bias is the starting value of the sums -- one load per channel and workgroup, handed out through
    // LDS -- and a per-pixel bias is requested straight into the sums before the first chunk: the loads land while the first
    // halo and slab do, and the epilogue is stores only. (Requested in the epilogue, one 32 x 32 unit ahead of its stores,
    // a wave had 4 KB in flight per memory round trip: 16 x 3 x 224 x 224 -> 64 took 133 us against 56 us without the bias.)
    const bool pix_bias = PIXB && p.bias && !p.partial;
    if (!PIXB && p.bias && !p.partial) {
        float* lds_b = reinterpret_cast<float*>(lds_h);          // the halo area is free until the first store_halo
        if (tid < BN) {
            const int o = o_tile * BN + tid;
            lds_b[tid] = o < p.O ? p.bias[(long)b * p.bias_sn + (long)o * p.bias_sc] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < NO; i++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const floatx4 v = *reinterpret_cast<const floatx4*>(lds_b + (wn * NO + i) * 32 + g * 8 + lh * 4);
#pragma unroll
                for (int j = 0; j < 2; j++)
#pragma unroll
                    for (int e = 0; e < 4; e++) acc[i][j][g * 4 + e] = v[e];
            }
        __syncthreads();                                        // read before the first halo lands in the same bytes
    }
    if (pix_bias) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int px = (wm * 2 + j) * 32 + li;
            const int ho = ho0 + (px >> p.sw_log), wo = wo0 + (px & (SW - 1));
            const float* bp = p.bias + (long)b * p.bias_sn + ((ho < p.Ho && wo < p.Wo) ? ((long)ho * p.Wo + wo) * p.bias_sp : 0);
#pragma unroll
            for (int i = 0; i < NO; i++) {
                const int o_base = o_tile * BN + (wn * NO + i) * 32 + lh * 4;
#pragma unroll
                for (int rr = 0; rr < 16; rr++) {
                    const int o = o_base + (rr >> 2) * 8 + (rr & 3);
                    acc[i][j][rr] = bp[(long)(o < p.O ? o : 0) * p.bias_sc];      // clamped: positions outside are never stored
                }
            }
        }
    }
    for (int chunk = chunk_lo; chunk < chunk_hi; chunk++) {
        store_halo(chunk);                                      // registers (chunk) -> LDS, fp16 channel-last
        __builtin_amdgcn_s_waitcnt(0x0070 | 0x0F00);            // vmcnt(0): this wave's slab pieces landed
        __syncthreads();
        load_halo(chunk + 1 < chunk_hi ? chunk + 1 : chunk);    // lands while the MFMAs below run (the last: once more, unused)
        // two fragment sets: the reads of tap t + 1 are issued before the MFMAs of tap t. A step's CPB planes and slabs
        // follow each other as one run of CPB * taps positions (plane, kernel row, kernel column).
        half8_t wf_[2][NO], pf_[2][2];
        auto fragments = [&](const int pl, const int tap, const int r, const int sx, const int set) {
            const int w_at = (CPB > 1 ? pl * p.slab_bytes : 0) + tap * 32;
            const char* hp = lds_h + (CPB > 1 ? pl * p.halo_plane : 0);
#pragma unroll
            for (int i = 0; i < NO; i++) wf_[set][i] = *reinterpret_cast<const half8_t*>(wrow[i] + w_at);
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int col = pcol[j] + sx;
                pf_[set][j] = *reinterpret_cast<const half8_t*>(hp + ((prow[j] + r) * p.pw + col) * 32 + ((lh ^ ((col >> 3) & 1)) << 4));
            }
        };
        int pl = 0, tp_ = 0, r = 0, sx = 0;                      // the position whose fragments were requested last
        auto next_position = [&]() {
            tp_++;
            if (++sx == p.Kw) { sx = 0; r++; }
            if (tp_ == taps) { tp_ = 0; r = 0; sx = 0; pl++; }
        };
        const int positions = CPB * taps;
        fragments(0, 0, 0, 0, 0);
        for (int pos = 0; pos < positions; pos += 2) {
            if (pos + 1 < positions) {
                next_position();
                fragments(pl, tp_, r, sx, 1);
            }
#pragma unroll
            for (int i = 0; i < NO; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf_[0][i], pf_[0][j], acc[i][j], 0, 0, 0);
            if (pos + 1 < positions) {
                if (pos + 2 < positions) {
                    next_position();
                    fragments(pl, tp_, r, sx, 0);
                }
#pragma unroll
                for (int i = 0; i < NO; i++)
#pragma unroll
                    for (int j = 0; j < 2; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf_[1][i], pf_[1][j], acc[i][j], 0, 0, 0);
            }
        }
        __syncthreads();                                        // everyone is done reading this chunk's LDS
        if (chunk + 1 < chunk_hi) load_slab(chunk + 1);
    }
    __builtin_amdgcn_s_waitcnt(0x0070 | 0x0F00);                // the halo requested once more after the last chunk

    // ---- epilogue: activation + NCHW store (lanes = adjacent pixels), or the bare sums of this channel group ----
    const long hw_out = (long)p.Ho * p.Wo;
    if (p.partial) {
        float* pb = p.partial + ((long)group * (gridDim.z / p.chunk_groups) + b) * p.O * hw_out;
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int px = (wm * 2 + j) * 32 + li;
            const int ho = ho0 + (px >> p.sw_log), wo = wo0 + (px & (SW - 1));
            if (ho >= p.Ho || wo >= p.Wo) continue;
            const long pix = (long)ho * p.Wo + wo;
#pragma unroll
            for (int i = 0; i < NO; i++) {
                const int o_base = o_tile * BN + (wn * NO + i) * 32 + lh * 4;
#pragma unroll
                for (int rr = 0; rr < 16; rr++) {
                    const int o = o_base + (rr >> 2) * 8 + (rr & 3);
                    if (o < p.O) pb[(long)o * hw_out + pix] = acc[i][j][rr];
                }
            }
        }
        return;
    }
    float* yb = p.y + (long)b * p.O * p.Ho * p.Wo;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int px = (wm * 2 + j) * 32 + li;
        const int ho = ho0 + (px >> p.sw_log), wo = wo0 + (px & (SW - 1));
        const bool px_ok = ho < p.Ho && wo < p.Wo;
        const long pix = px_ok ? (long)ho * p.Wo + wo : 0;
#pragma unroll
        for (int i = 0; i < NO; i++) {
            const int o_base = o_tile * BN + (wn * NO + i) * 32 + lh * 4;
#pragma unroll
            for (int rr = 0; rr < 16; rr++) {
                const int o = o_base + (rr >> 2) * 8 + (rr & 3);
                float v = acc[i][j][rr];
                if (p.relu) v = v > 0.f ? v : 0.f;
                if (px_ok && o < p.O) yb[(long)o * hw_out + pix] = v;
            }
        }
    }
}

// y = act(bias + the channel groups' sums, added in ascending group order)
__global__ __launch_bounds__(256) void conv_group_sum_kernel(float* __restrict__ y, const float* __restrict__ partial, const float* __restrict__ bias,
                                                             int groups, int O, long hw, long per_group, long bias_sp, long bias_sc,
                                                             long bias_sn, int relu) {
    const long t = (long)blockIdx.x * 256 + threadIdx.x;        // element of y: (image, channel, pixel)
    if (t >= per_group) return;
    float v = 0.f;
    for (int g = 0; g < groups; g++) v += partial[(long)g * per_group + t];
    if (bias) {
        const long pix = t % hw, bo = t / hw;
        v += bias[(bo / O) * bias_sn + pix * bias_sp + (bo % O) * bias_sc];
    }
    if (relu) v = v > 0.f ? v : 0.f;
    y[t] = v;
}

static bool conv_igemm_gen_applicable(const float* x, size_t C, size_t H, size_t W, size_t O, size_t K_h, size_t K_w, size_t stride,
                                      size_t pad, size_t N) {
    (void)O;
    // (a strided 1x1 convolution has one tap per chunk to multiply between two barriers: its column matrix is the cheaper way)
    (void)x; (void)W;
    return C >= 1 && stride <= 4 && K_h * K_w >= 2 && K_h * K_w <= 64 && pad < 0x10000 &&
           N <= 65535 && H * W < 0x7fffffffull && C * H * W < 0x7fffffffull;
}

// The segment width of the any-geometry kernel: the power of two >= 16 that covers the output width, or, when the slab
// and the halo of that tile do not fit LDS or a thread's staging share, the widest narrower one that does (more rows of
// fewer columns: 7x7 stride 2 on 112 output columns takes 4 x 64 instead of 2 x 128 pixels). Returns log2 of the
// width, 0 when nothing fits. Sized for the larger channel tile; the launch may still pick the smaller one.
static int conv_igemm_gen_sw_log(size_t W_out, size_t O, size_t K_h, size_t K_w, size_t stride, size_t pad) {
    const int taps = (int)(K_h * K_w);
    int sw_log = 8;
    while (sw_log > 4 && (size_t)(1 << (sw_log - 1)) >= W_out) sw_log--;
    const int shift = (int)(((4 - (long)(pad % 4)) % 4 + 4) % 4);
    const int BN = O > 64 ? 128 : 64;
    const size_t slab = (size_t)BN * (taps * 32 + 16);
    for (; sw_log >= 4; sw_log--) {
        const int SW = 1 << sw_log, SR = CG_PX / SW;
        const int span = (int)((SR - 1) * stride + K_h);
        int pw = (int)((SW - 1) * stride + K_w) + shift;
        pw = (pw + 3) / 4 * 4;
        if ((slab + 1023) / 1024 * 1024 + (size_t)span * pw * 32 <= 160 * 1024 - 512 &&
            (size_t)2 * span * (pw / 4) <= (size_t)CG_THREADS * CG_TP_MAX)
            return sw_log;
    }
    return 0;
}
static bool conv_igemm_gen_fits(size_t W_out, size_t O, size_t K_h, size_t K_w, size_t stride, size_t pad) {
    return conv_igemm_gen_sw_log(W_out, O, K_h, K_w, stride, pad) != 0;
}

// Returns NZHIP_E_UNSUPPORTED (nothing enqueued, no error text) when the tile does not fit LDS or a thread's staging share.
// dst[row][0 .. Ww) = src[row][0 .. W) followed by zeros, Ww the next multiple of 4: image rows that are whole 16-byte
// pieces. The zeros stand where the convolution's padding would: the kernel below then reads columns W .. Ww - 1 as
// zeros from memory instead of as zeros from its bounds check, and the output extents stay what they were.
// 256 >> wq_log rows per workgroup, a thread four columns of a row.
__global__ __launch_bounds__(256) void widen_rows_kernel(float* __restrict__ dst, const float* __restrict__ src, long rows, int W, int Ww,
                                                         int wq_log) {
    const long row = (long)blockIdx.x * (256 >> wq_log) + (threadIdx.x >> wq_log);
    if (row >= rows) return;
    const float* srow = src + row * W;
    float* drow = dst + row * Ww;
    for (int w0 = (threadIdx.x & ((1 << wq_log) - 1)) * 4; w0 < Ww; w0 += 4 << wq_log) {
        floatx4 v;
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = w0 + j < W ? srow[w0 + j] : 0.f;
        *reinterpret_cast<floatx4*>(drow + w0) = v;
    }
}
// *out: a pooled workspace holding `rows` rows of src widened from W to the next multiple of 4 columns
static int widen_rows(float** out, const float* src, size_t rows, size_t W, hipStream_t s) {
    const size_t Ww = (W + 3) / 4 * 4;
    int wq_log = 0;
    while (wq_log < 8 && ((size_t)4 << wq_log) < Ww) wq_log++;
    const size_t blocks = (rows + (256 >> wq_log) - 1) / (256 >> wq_log);
    if (blocks > 0x7fffffffull || Ww >= 0x3fffffff) return set_error(NZHIP_E_UNSUPPORTED, "widen_rows: extents beyond the kernel's grid");
    if (int rc = workspace_alloc(reinterpret_cast<void**>(out), rows * Ww * sizeof(float), s)) return rc;
    hipLaunchKernelGGL(widen_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, s, *out, src, (long)rows, (int)W, (int)Ww, wq_log);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        workspace_free(*out, s);
        *out = nullptr;
        return set_hip_error(e, "widen_rows kernel launch");
    }
    return NZHIP_OK;
}

// 1x1 layers are products whose operands have an image's pixels as their contiguous rows: with a pixel count that is not
// a multiple of 4 (7 x 7, 17 x 17, 35 x 35 images) the product loads them element by element. A zero-filled copy with
// planes of the next multiple of 4 pays for itself when the copied operand is the small one of the product, i.e. when
// every copied element takes part in many multiply-adds (`flops_per_element`: 2 x the channels on the other side):
// 16 x 512 x 7 x 7 -> 2048 forward 40 -> 25 us, its data gradient 47 -> 29; 16 x 192 x 35 x 35 -> 64 forward would go from
// 22 to 33 us (the copy of x costs what the whole product does) and stays as it is.
static bool conv1x1_wants_wide_planes(size_t HW, double flops, double flops_per_element) {
    const char* widen_env = getenv("NZHIP_CONV_WIDEN");              // benchmarks and tests: 0 never, 1 always (read per call)
    if (HW % 4 == 0) return false;
    return widen_env ? atoi(widen_env) != 0 : (flops >= 4e8 && flops_per_element >= 512.0);
}

static int conv_igemm_gen_launch(float* y, const float* x, const float* w_ref, const float* bias, size_t N, size_t C, size_t H,
                                 size_t W, size_t O, size_t K_h, size_t K_w, size_t stride, size_t pad, size_t w_batch,
                                 int64_t bias_sp, int64_t bias_sc, int64_t bias_sn, int act, size_t H_out, size_t W_out,
                                 bool w_mirror, hipStream_t s) {
    const int taps = (int)(K_h * K_w);
    const int sw_log = conv_igemm_gen_sw_log(W_out, O, K_h, K_w, stride, pad);
    if (sw_log == 0) return NZHIP_E_UNSUPPORTED;
    const int SW = 1 << sw_log, SR = CG_PX / SW;
    // 128 output channels per workgroup, unless that leaves compute units without one (16 x 128 x 56 x 56 -> 128 at
    // stride 2: 64 workgroups; with 64-channel tiles 128 of them, 40 against 49 us)
    static const char* bn_env = getenv("NZHIP_CONV_BN");            // benchmarking only
    const size_t groups128 = N * ((H_out + SR - 1) / SR) * ((W_out + SW - 1) / SW) * ((O + 127) / 128);
    const int BN = bn_env ? (atoi(bn_env) == 128 ? 128 : 64) : (O > 64 && groups128 >= (size_t)device_cu_count() ? 128 : 64);
    const int shift = (int)(((4 - (long)(pad % 4)) % 4 + 4) % 4);   // staged column 0 is a multiple of four image columns
    const int span = (int)((SR - 1) * stride + K_h);
    int pw = (int)((SW - 1) * stride + K_w) + shift;
    pw = (pw + 3) / 4 * 4;
    const int w_pitch = taps * 32 + 16, slab_bytes = BN * w_pitch;
    const int halo_off = (slab_bytes + 1023) / 1024 * 1024;
    const size_t lds_need = (size_t)halo_off + (size_t)span * pw * 32;
    const size_t tasks = (size_t)2 * span * (pw / 4);
    if (lds_need > 160 * 1024 - 512 || tasks > (size_t)CG_THREADS * CG_TP_MAX) return NZHIP_E_UNSUPPORTED;
    const int n_chunks = (int)((C + IG_CC - 1) / IG_CC), n_otiles = (int)((O + BN - 1) / BN);
    const size_t seg_rows = (H_out + SR - 1) / SR, segs_w = (W_out + SW - 1) / SW;
    if (n_otiles > 65535 || seg_rows * segs_w > 0x7fffffffull) return NZHIP_E_UNSUPPORTED;
    // Few segments and many channels (deep layers on small images): the contraction is split over groups of at least
    // two channel chunks until every compute unit has a workgroup; a second kernel adds the groups' sums in order.
    int chunk_groups = 1, chunks_per_group = n_chunks;
    {
        const size_t wgs = N * seg_rows * segs_w * n_otiles, cus = (size_t)device_cu_count();
        if (wgs < cus && n_chunks >= 4) {
            size_t want = (cus + wgs - 1) / wgs;
            if (want > (size_t)n_chunks / 2) want = (size_t)n_chunks / 2;
            chunks_per_group = (int)((n_chunks + want - 1) / want);
            chunk_groups = (n_chunks + chunks_per_group - 1) / chunks_per_group;
        }
        if (N * (size_t)chunk_groups > 65535) return NZHIP_E_UNSUPPORTED;
    }
    // Two chunks per loop step (the store / barrier / request phases paid half as often) when the contraction is long and
    // not split, the rows allow 16-byte loads and two slabs and two halo planes fit LDS and a thread's staging share;
    // the weight image then holds an even number of slabs per channel tile, the last one zero when n_chunks is odd.
    static const char* cpb_env = getenv("NZHIP_CONV_CPB");           // benchmarking only: 1 keeps one chunk per step
    // Rows that are not whole 16-byte pieces (14-, 30-, 35-wide images) stage with four loads and four bounds per task
    // and never two chunks per step. From about 8 GFLOP on, a zero-filled copy with rows of the next multiple of 4 pays
    // for itself (16 x 192 x 35 x 35 -> 192: 120 -> 81 us; 16 x 512 x 14 x 14 -> 512: 85 -> 70; 16 x 256 x 14 x 14 -> 256
    // would stay at 37).
    const char* widen_env = getenv("NZHIP_CONV_WIDEN");              // benchmarks and tests: 0 never, 1 wherever rows are not whole pieces (read per call)
    float* x_wide = nullptr;
    const double flops = 2.0 * (double)N * (double)H_out * (double)W_out * (double)C * (double)taps * (double)O;
    if (W % 4 != 0 && (widen_env ? atoi(widen_env) != 0 : flops >= 8e9)) {
        const size_t Ww = (W + 3) / 4 * 4;
        if (C * H * Ww < 0x7fffffffull && N * C * H < 0x7fffffffull) {      // the kernels' int offsets and grids
            if (int rc = widen_rows(&x_wide, x, N * C * H, W, s)) return rc;
            x = x_wide;
            W = Ww;
        }
    }
    const bool vec = W % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0;
    const bool two = vec && chunk_groups == 1 && n_chunks >= 4 && !(cpb_env && atoi(cpb_env) == 1) &&
                     ((size_t)2 * slab_bytes + 1023) / 1024 * 1024 + (size_t)2 * span * pw * 32 <= 160 * 1024 - 512 &&
                     2 * tasks <= (size_t)CG_THREADS * CG_TP_MAX;
    const int cpb = two ? 2 : 1;
    const int img_chunks = (n_chunks + cpb - 1) / cpb * cpb;
    const size_t image_bytes = (size_t)n_otiles * img_chunks * slab_bytes, bytes = image_bytes * w_batch;
    uint64_t key[PREPARED_KEY_WORDS];
    conv_image_key(key, 3, (int)K_h, (int)K_w, BN, w_ref, C, O, img_chunks, n_otiles, w_batch, w_mirror);
    ImageLease lease;
    if (int rc = image_acquire(PREPARED_CONV_W, key, bytes, s, &lease)) {
        if (x_wide) workspace_free(x_wide, s);
        return rc;
    }
    _Float16* wimg = static_cast<_Float16*>(lease.ptr);
    if (lease.fill) {
        dim3 pg((unsigned)((BN * taps + 255) / 256), (unsigned)(w_batch * n_otiles * img_chunks));
        hipLaunchKernelGGL(conv_weight_image_gen_kernel, pg, dim3(256), 0, s, wimg, w_ref, (int)C, (int)O, taps, BN, w_pitch / 2,
                           img_chunks, n_otiles, w_mirror ? 1 : 0);
    }
    ConvGenArgs a;
    a.y = y; a.x = x; a.wimg = wimg; a.bias = bias;
    a.C = (int)C; a.H = (int)H; a.W = (int)W; a.O = (int)O; a.Ho = (int)H_out; a.Wo = (int)W_out;
    a.Kh = (int)K_h; a.Kw = (int)K_w; a.stride = (int)stride; a.pad = (int)pad;
    a.n_chunks = n_chunks; a.n_otiles = n_otiles; a.w_batched = w_batch > 1;
    a.sw_log = sw_log; a.span = span; a.pw = pw; a.shift = shift; a.segs_w = (int)segs_w;
    a.w_pitch = w_pitch; a.slab_bytes = slab_bytes; a.halo_off = halo_off;
    a.bias_sp = bias_sp; a.bias_sc = bias_sc; a.bias_sn = bias_sn; a.relu = act == NZHIP_ACT_RELU;
    a.chunk_groups = chunk_groups; a.chunks_per_group = chunks_per_group; a.partial = nullptr;
    a.img_chunks = img_chunks; a.halo_plane = span * pw * 32;
    static const char* bias_map_env = getenv("NZHIP_CONV_BIAS_MAP");   // benchmarking only: 0 keeps the image-major order
    a.bias_map = !(bias_map_env && atoi(bias_map_env) == 0) && N >= 2;
    size_t lds_use = lds_need;
    if (two) {                                                       // the kernel counts steps of two chunks
        a.n_chunks = img_chunks / 2; a.chunks_per_group = a.n_chunks;
        a.halo_off = (2 * slab_bytes + 1023) / 1024 * 1024;
        lds_use = (size_t)a.halo_off + (size_t)2 * a.halo_plane;
    }
    const size_t per_group = N * O * H_out * W_out;
    float* partial = nullptr;
    if (chunk_groups > 1) {
        if (int rc = workspace_alloc(reinterpret_cast<void**>(&partial), (size_t)chunk_groups * per_group * sizeof(float), s)) {
            image_release(lease, s, true);
            if (x_wide) workspace_free(x_wide, s);
            return rc;
        }
        a.partial = partial;
    }
    const int tp = (int)((cpb * tasks + CG_THREADS - 1) / CG_THREADS);
    auto pick = [&](auto vec_tag, auto pix_tag, auto cpb_tag) {
        constexpr bool V = decltype(vec_tag)::value, P = decltype(pix_tag)::value;
        constexpr int B = decltype(cpb_tag)::value;
        return BN == 128 ? (tp <= 1   ? conv_igemm_gen_kernel<2, 1, V, P, B>
                            : tp == 2 ? conv_igemm_gen_kernel<2, 2, V, P, B>
                                      : conv_igemm_gen_kernel<2, 3, V, P, B>)
                         : (tp <= 1   ? conv_igemm_gen_kernel<1, 1, V, P, B>
                            : tp == 2 ? conv_igemm_gen_kernel<1, 2, V, P, B>
                                      : conv_igemm_gen_kernel<1, 3, V, P, B>);
    };
    using one_t = std::integral_constant<int, 1>;
    using two_t = std::integral_constant<int, 2>;
    const bool pixb = bias && bias_sp != 0 && chunk_groups == 1;
    auto kfn = two   ? (pixb ? pick(std::true_type{}, std::true_type{}, two_t{}) : pick(std::true_type{}, std::false_type{}, two_t{}))
               : vec ? (pixb ? pick(std::true_type{}, std::true_type{}, one_t{}) : pick(std::true_type{}, std::false_type{}, one_t{}))
                     : (pixb ? pick(std::false_type{}, std::true_type{}, one_t{}) : pick(std::false_type{}, std::false_type{}, one_t{}));
    int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kfn), (int)lds_use, "hipFuncSetAttribute(conv_igemm_gen)");
    if (rc == NZHIP_OK) {
        hipLaunchKernelGGL(kfn, dim3((unsigned)(seg_rows * segs_w), (unsigned)n_otiles, (unsigned)(N * chunk_groups)), dim3(CG_THREADS),
                           lds_use, s, a);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) rc = set_hip_error(e, "conv_igemm_gen kernel launch");
    }
    if (rc == NZHIP_OK && partial) {
        hipLaunchKernelGGL(conv_group_sum_kernel, dim3((unsigned)((per_group + 255) / 256)), dim3(256), 0, s, y, partial, bias, chunk_groups,
                           (int)O, (long)(H_out * W_out), (long)per_group, (long)bias_sp, (long)bias_sc, (long)bias_sn,
                           act == NZHIP_ACT_RELU ? 1 : 0);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) rc = set_hip_error(e, "conv_group_sum kernel launch");
    }
    const int rc3 = partial ? workspace_free(partial, s) : NZHIP_OK;
    const int rc2 = image_release(lease, s, rc == NZHIP_OK);
    const int rc4 = x_wide ? workspace_free(x_wide, s) : NZHIP_OK;
    return rc ? rc : (rc2 ? rc2 : (rc3 ? rc3 : rc4));
}

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

// ---- weight gradient of the 3x3, stride 1, pad 1 convolution without a column matrix ----------------
//   dW[(c, r, s)][o] += sum over n, h, w of f16(x[n][c][h+r-1][w+s-1]) * f16(dy[n][o][h][w])
// As a GEMM the contraction runs over pixels, and both operands already are pixel-contiguous in NCHW.
// A workgroup owns 32 input channels x 128 output channels (9 x 4 blocks of 32x32, one column of blocks
// per wave) and a band of rows of one image. Per row and 128-pixel segment it keeps in LDS
//   * the dy row, fp16, [o][pixel];
//   * the x rows h-1, h, h+1 (a rolling window of three), each as THREE copies shifted by s-1 pixels, so
//     that every tap reads 16-byte aligned runs of 8 pixels. The copies are made in registers: a lane holds
//     8 adjacent pixels, takes the pixel to its left / right from the neighbouring lane (DPP row shift; the
//     first and last lane of a row of 16 load it) and funnel-shifts.
// Next row's operands are requested into registers before the MFMA phase. Partial sums of the row bands go to
// a workspace and are added in a fixed order by conv_dw_reduce_kernel.
constexpr int DW_CC = 32, DW_OT = 128, DW_PX = 128, DW_PITCH = DW_PX * 2 + 16;      // LDS row pitch in bytes
constexpr int DW_XS_BYTES = 3 * 3 * DW_CC * DW_PITCH, DW_ZS_BYTES = DW_OT * DW_PITCH;

struct ConvDwArgs {
    const float* x;        // [N, C, H, W]
    const float* dy;       // [N, O, H, W]
    float* partial;        // [chunk][o_tile][image][band][rows = nch*9][ncols]
    int C, H, W, O;
    int bands, band_rows;  // row bands per image and rows per band
    int n_images;
};

// VEC: W is a multiple of 8 and x, dy are 16-byte aligned (two 16-byte loads per group of 8 pixels); otherwise
// every pixel is loaded and bounds-checked on its own.
template <bool VEC>
__global__ __launch_bounds__(256) void conv_dw_kernel(const ConvDwArgs p) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    char* xs = lds;                       // [slot 3][shift 3][channel 32] rows of DW_PITCH bytes
    char* zs = lds + DW_XS_BYTES;         // [o 128] rows of DW_PITCH bytes
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lh = lane >> 5;
    const int band = blockIdx.x % p.bands, img = blockIdx.x / p.bands;
    const int c0 = blockIdx.y * DW_CC, o0 = blockIdx.z * DW_OT;
    const int nch = (p.C - c0) < DW_CC ? (p.C - c0) : DW_CC;
    const int ncols = (p.O - o0) < DW_OT ? (p.O - o0) : DW_OT;
    const int h_begin = band * p.band_rows;
    const int h_end = (h_begin + p.band_rows) < p.H ? (h_begin + p.band_rows) : p.H;
    const long plane = (long)p.H * p.W;
    const float* ximg = p.x + ((long)img * p.C + c0) * plane;
    const float* zimg = p.dy + ((long)img * p.O + o0) * plane;

    floatx16 acc[9];
#pragma unroll
    for (int t = 0; t < 9; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[t][r] = 0.f;

    // staging tasks: x row = 32 channels x 16 groups of 8 pixels (two per thread: channels tid/16 and 16 + tid/16);
    // dy row = 128 output channels x 16 groups (eight per thread)
    const int g = tid & 15;
    float xr[2][8], xl[2], xrt[2];        // a task's 8 pixels, the pixel left of them, the pixel right of them
    float zr[8][8];

    auto load_x = [&](int h, int w0) {
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int c = u * 16 + (tid >> 4);
            const int w = w0 + g * 8;
            const bool ok = c < nch && h >= 0 && h < p.H && w < p.W;       // VEC: a group is wholly inside or outside
            const float* src = ximg + (long)c * plane + (long)h * p.W + w;
#pragma unroll
            for (int e = 0; e < 8; e++) xr[u][e] = 0.f;
            xl[u] = 0.f;
            xrt[u] = 0.f;
            if (ok) {
                if (VEC) {
                    const floatx4 a = *reinterpret_cast<const floatx4*>(src), b = *reinterpret_cast<const floatx4*>(src + 4);
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        xr[u][e] = a[e];
                        xr[u][4 + e] = b[e];
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 8; e++)
                        if (w + e < p.W) xr[u][e] = src[e];
                }
                if (g == 0 && w > 0) xl[u] = src[-1];
                if (g == 15 && w + 8 < p.W) xrt[u] = src[8];
            }
        }
    };
    auto load_z = [&](int h, int w0) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int o = i * 16 + (tid >> 4);
            const int w = w0 + g * 8;
            const bool ok = o < ncols && h < p.H && w < p.W;
            const float* src = zimg + (long)o * plane + (long)h * p.W + w;
#pragma unroll
            for (int e = 0; e < 8; e++) zr[i][e] = 0.f;
            if (ok) {
                if (VEC) {
                    const floatx4 a = *reinterpret_cast<const floatx4*>(src), b = *reinterpret_cast<const floatx4*>(src + 4);
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        zr[i][e] = a[e];
                        zr[i][4 + e] = b[e];
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 8; e++)
                        if (w + e < p.W) zr[i][e] = src[e];
                }
            }
        }
    };
    auto pack2 = [](float lo, float hi) -> unsigned {
        const _Float16 a = (_Float16)lo, b = (_Float16)hi;
        return (unsigned)__builtin_bit_cast(unsigned short, a) | ((unsigned)__builtin_bit_cast(unsigned short, b) << 16);
    };
    typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
    auto store_x = [&](int slot) {
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int c = u * 16 + (tid >> 4);
            const unsigned p0 = pack2(xr[u][0], xr[u][1]), p1 = pack2(xr[u][2], xr[u][3]), p2 = pack2(xr[u][4], xr[u][5]),
                           p3 = pack2(xr[u][6], xr[u][7]);
            // neighbour pixels: from the lane one group to the left / right inside the row of 16 lanes;
            // the outermost lanes keep the pixel they loaded themselves
            const unsigned left = (unsigned)__builtin_amdgcn_update_dpp((int)pack2(0.f, xl[u]), (int)p3, 0x111, 0xf, 0xf, false);
            const unsigned right = (unsigned)__builtin_amdgcn_update_dpp((int)pack2(xrt[u], 0.f), (int)p0, 0x101, 0xf, 0xf, false);
            const uintx4 sm = {__builtin_amdgcn_alignbit(p0, left, 16), __builtin_amdgcn_alignbit(p1, p0, 16),
                               __builtin_amdgcn_alignbit(p2, p1, 16), __builtin_amdgcn_alignbit(p3, p2, 16)};   // x[w-1]
            const uintx4 s0 = {p0, p1, p2, p3};                                                                  // x[w]
            const uintx4 sp = {__builtin_amdgcn_alignbit(p1, p0, 16), __builtin_amdgcn_alignbit(p2, p1, 16),
                               __builtin_amdgcn_alignbit(p3, p2, 16), __builtin_amdgcn_alignbit(right, p3, 16)}; // x[w+1]
            char* base = xs + ((slot * 3) * DW_CC + c) * DW_PITCH + g * 16;
            *reinterpret_cast<uintx4*>(base) = sm;
            *reinterpret_cast<uintx4*>(base + DW_CC * DW_PITCH) = s0;
            *reinterpret_cast<uintx4*>(base + 2 * DW_CC * DW_PITCH) = sp;
        }
    };
    auto store_z = [&]() {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int o = i * 16 + (tid >> 4);
            const uintx4 v = {pack2(zr[i][0], zr[i][1]), pack2(zr[i][2], zr[i][3]), pack2(zr[i][4], zr[i][5]),
                              pack2(zr[i][6], zr[i][7])};
            *reinterpret_cast<uintx4*>(zs + o * DW_PITCH + g * 16) = v;
        }
    };

    for (int w0 = 0; w0 < p.W; w0 += DW_PX) {
        // rows h_begin - 1 and h_begin of this segment go into their slots, then row h_begin + 1 and the
        // first dy row wait in registers like in every later iteration
        __syncthreads();                                       // the previous segment's readers are done
        load_x(h_begin - 1, w0);
        store_x((h_begin + 2) % 3);                            // slot of row h: (h + 3) % 3, here h = h_begin - 1
        load_x(h_begin, w0);
        store_x(h_begin % 3);
        load_x(h_begin + 1, w0);
        load_z(h_begin, w0);
        for (int h = h_begin; h < h_end; h++) {
            store_x((h + 1) % 3);
            store_z();
            __syncthreads();
            load_x(h + 2, w0);                                 // past the image: zeros; past the band's last use: never read
            load_z(h + 1 < h_end ? h + 1 : p.H, w0);
            const char* zrow = zs + (wave * 32 + li) * DW_PITCH + lh * 16;
#pragma unroll 2
            for (int j = 0; j < DW_PX / 16; j++) {
                const half8_t bfrag = *reinterpret_cast<const half8_t*>(zrow + j * 32);
#pragma unroll
                for (int r = 0; r < 3; r++) {
                    const int slot = (h + r + 2) % 3;          // row h + r - 1
                    const char* arow = xs + ((slot * 3) * DW_CC + li) * DW_PITCH + lh * 16 + j * 32;
#pragma unroll
                    for (int sx = 0; sx < 3; sx++) {
                        const half8_t afrag = *reinterpret_cast<const half8_t*>(arow + sx * DW_CC * DW_PITCH);
                        acc[r * 3 + sx] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afrag, bfrag, acc[r * 3 + sx], 0, 0, 0);
                    }
                }
            }
            __syncthreads();                                   // before zs and the oldest x slot are overwritten
        }
    }

    // partial sums of this band: rows (c, tap) in the order of dW, columns o
    const long region = (long)DW_CC * 9 * DW_OT;
    float* P = p.partial + ((((long)blockIdx.y * gridDim.z + blockIdx.z) * p.n_images + img) * p.bands + band) * region;
    const int o = wave * 32 + li;
#pragma unroll
    for (int t = 0; t < 9; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int c = (r >> 2) * 8 + lh * 4 + (r & 3);
            if (c < nch && o < ncols) P[(long)(c * 9 + t) * ncols + o] = acc[t][r];
        }
}

// dW[b][(c0 + c)*9 + t][o0 + o] += sum over the S partial regions of image group b, in ascending order.
// b: one index per weight copy (per-sample weights: S = bands of that image; shared weights: S = images x bands).
__global__ __launch_bounds__(256) void conv_dw_reduce_kernel(float* __restrict__ dW, const float* __restrict__ P, int S,
                                                             int C, int O, int n_otiles, long group_stride_P,
                                                             long group_stride_dW) {
    // 32 outputs per workgroup, eight threads per output: thread q adds the regions of its contiguous
    // eighth in ascending order, then the eight sums are added in ascending q
    __shared__ float part[8][32];
    const int chunk = blockIdx.y / n_otiles, ot = blockIdx.y % n_otiles, b = blockIdx.z;
    const int c0 = chunk * DW_CC, o0 = ot * DW_OT;
    const int nch = (C - c0) < DW_CC ? (C - c0) : DW_CC;
    const int ncols = (O - o0) < DW_OT ? (O - o0) : DW_OT;
    const int q = threadIdx.x >> 5, tl = threadIdx.x & 31;
    const int t = blockIdx.x * 32 + tl;
    const bool live = t < nch * 9 * ncols;
    const long region = (long)DW_CC * 9 * DW_OT;
    const float* src = P + ((long)blockIdx.y * gridDim.z + b) * group_stride_P + t;
    const int per = (S + 7) / 8, s0 = q * per, s1 = (s0 + per) < S ? (s0 + per) : S;
    float sum = 0.f;
    if (live)
        for (int s = s0; s < s1; s++) sum += src[(long)s * region];
    part[q][tl] = sum;
    __syncthreads();
    if (q != 0 || !live) return;
#pragma unroll
    for (int k = 1; k < 8; k++) sum += part[k][tl];
    const int row = t / ncols, col = t % ncols;
    dW[(long)b * group_stride_dW + ((long)c0 * 9 + row) * O + o0 + col] += sum;
}

// The same sums for at most 8 regions per weight copy (per-sample weights: the bands of one image): one thread per
// output adds them in ascending order -- with at most one region per eighth that is the order of the kernel above --
// and a wave reads 256 contiguous bytes of every region (16 x 64 x 128 x 128 -> 128 with a weight copy per image: 38 MB of
// partial sums, 22.7 -> 10 us).
__global__ __launch_bounds__(256) void conv_dw_reduce_few_kernel(float* __restrict__ dW, const float* __restrict__ P, int S,
                                                                 int C, int O, int n_otiles, long group_stride_P,
                                                                 long group_stride_dW) {
    const int chunk = blockIdx.y / n_otiles, ot = blockIdx.y % n_otiles, b = blockIdx.z;
    const int c0 = chunk * DW_CC, o0 = ot * DW_OT;
    const int nch = (C - c0) < DW_CC ? (C - c0) : DW_CC;
    const int ncols = (O - o0) < DW_OT ? (O - o0) : DW_OT;
    const int t = blockIdx.x * 256 + threadIdx.x;
    if (t >= nch * 9 * ncols) return;
    const long region = (long)DW_CC * 9 * DW_OT;
    const float* src = P + ((long)blockIdx.y * gridDim.z + b) * group_stride_P + t;
    float v[8];
#pragma unroll
    for (int s = 0; s < 8; s++) v[s] = src[(long)(s < S ? s : 0) * region];      // all requests first
    float sum = 0.f;
#pragma unroll
    for (int s = 0; s < 8; s++)
        if (s < S) sum += v[s];
    const int row = t / ncols, col = t % ncols;
    dW[(long)b * group_stride_dW + ((long)c0 * 9 + row) * O + o0 + col] += sum;
}

// ---- weight gradient of the 3x3, stride 1, pad 1 convolution with a handful of channels -------------
// With C <= 4 and O <= 2 the gradient has at most 72 entries per weight copy, each a sum over every pixel:
// a stream over x and dy, not a matrix product. Same thread mapping as the forward stream kernel (a lane
// owns 4 adjacent columns of a 16-row strip, three rounded x rows in a rolling register window, halo
// columns from the neighbour lanes), and C*9*O running sums per lane:
//     acc[(c, r, s)][o] += f16(x[c][h + r - 1][w + s - 1]) * f16(dy[o][h][w]).
// A wave adds its lanes in a fixed tree and writes one partial vector per strip; small_dw_reduce_kernel
// adds the strips (and, for shared weights, the images) in ascending order.
template <int O_T, int C_T>
__global__ __launch_bounds__(256) void conv3x3_dw_stream_kernel(float* __restrict__ partial, const float* __restrict__ x,
                                                                const float* __restrict__ dy, int H, int W) {
    constexpr int Q = C_T * 9 * O_T;
    int bx, by, b;
    xcd_contiguous_block(bx, by, b);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int w0 = (bx * 64 + lane) * 4;
    const int strip = by * 4 + wave, n_strips = gridDim.y * 4;
    const int h0 = strip * ST_ROWS;
    float acc[Q];
#pragma unroll
    for (int q = 0; q < Q; q++) acc[q] = 0.f;
    if (h0 < H) {                                                // uniform over the wave
        const bool col_ok = w0 < W;                              // W % 4 == 0: a lane's quad is all in or all out
        const int wq = col_ok ? w0 : 0;
        const bool has_l = col_ok && w0 > 0, has_r = col_ok && w0 + 4 < W;
        const int wx = lane == 0 ? (has_l ? w0 - 1 : wq) : (lane == 63 && has_r ? w0 + 4 : wq);
        const float* xb = x + (long)b * C_T * H * W;
        const float* gb = dy + (long)b * O_T * H * W;
        const long plane = (long)H * W;
        const int rows = (H - h0) < ST_ROWS ? (H - h0) : ST_ROWS;
        const int T = rows + 2;
        float win[3][C_T][6];
        for (int t0 = 0; t0 < T; t0 += 3) {
#pragma unroll
            for (int u = 0; u < 3; u++) {
                const int t = t0 + u;
                if (t >= T) break;
                const int hi = h0 - 1 + t;
                const bool in_img = hi >= 0 && hi < H;
                const float* row = xb + (long)(in_img ? hi : 0) * W;
#pragma unroll
                for (int c = 0; c < C_T; c++) {
                    const floatx4 qv = *reinterpret_cast<const floatx4*>(row + c * plane + wq);
                    const float ex = row[c * plane + wx];
                    float r5[5];
#pragma unroll
                    for (int e = 0; e < 4; e++) r5[e] = (in_img && col_ok) ? round_f16(qv[e]) : 0.f;
                    r5[4] = in_img ? round_f16(ex) : 0.f;
                    const float below = from_lane_below(r5[3]), above = from_lane_above(r5[0]);
                    win[u][c][0] = has_l ? (lane == 0 ? r5[4] : below) : 0.f;
#pragma unroll
                    for (int e = 0; e < 4; e++) win[u][c][1 + e] = r5[e];
                    win[u][c][5] = has_r ? (lane == 63 ? r5[4] : above) : 0.f;
                }
                if (t < 2) continue;
                const int ho = h0 + t - 2;                       // rows t-2, t-1, t are the window of output row ho
                float g[O_T][4];
#pragma unroll
                for (int o = 0; o < O_T; o++) {
                    const floatx4 gv = *reinterpret_cast<const floatx4*>(gb + (long)o * plane + (long)ho * W + wq);
#pragma unroll
                    for (int e = 0; e < 4; e++) g[o][e] = col_ok ? round_f16(gv[e]) : 0.f;
                }
#pragma unroll
                for (int c = 0; c < C_T; c++)
#pragma unroll
                    for (int r = 0; r < 3; r++) {
                        const int slot = (u + 1 + r) % 3;        // step t-2+r lives in slot (t-2+r) % 3, and t % 3 == u
#pragma unroll
                        for (int s2 = 0; s2 < 3; s2++)
#pragma unroll
                            for (int o = 0; o < O_T; o++)
#pragma unroll
                                for (int e = 0; e < 4; e++)
                                    acc[((c * 3 + r) * 3 + s2) * O_T + o] =
                                        __builtin_fmaf(win[slot][c][e + s2], g[o][e], acc[((c * 3 + r) * 3 + s2) * O_T + o]);
                    }
            }
        }
    }
    float* dst = partial + (((long)b * n_strips + strip) * gridDim.x + bx) * Q;
#pragma unroll
    for (int q = 0; q < Q; q++) {
        float v = acc[q];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off);
        if (lane == 0) dst[q] = v;
    }
}

// dW[g][q] += sum over the S partial vectors of group g (a weight copy), in a fixed order: eight threads per
// entry add a contiguous eighth each in ascending order, then the eight sums are added in ascending order.
__global__ __launch_bounds__(256) void small_dw_reduce_kernel(float* __restrict__ dW, const float* __restrict__ P, int S,
                                                              int Q) {
    __shared__ float part[8][32];
    const int k = threadIdx.x >> 5, tl = threadIdx.x & 31;
    const int q = blockIdx.x * 32 + tl, g = blockIdx.y;
    const bool live = q < Q;
    const float* src = P + (long)g * S * Q + q;
    const int per = (S + 7) / 8, s0 = k * per, s1 = (s0 + per) < S ? (s0 + per) : S;
    float sum = 0.f;
    if (live)
        for (int s = s0; s < s1; s++) sum += src[(long)s * Q];
    part[k][tl] = sum;
    __syncthreads();
    if (k != 0 || !live) return;
#pragma unroll
    for (int j = 1; j < 8; j++) sum += part[j][tl];
    dW[(long)g * Q + q] += sum;
}

// Gradient of the per-pixel, per-channel bias the reference's Conv2d adds to the matmul result ([1,1,HW,O]):
//   dbias[p][o] += sum over n of dz[n][o][p]   (dz in NCHW),
// i.e. Col2ImgNode::backward (a transpose of the whole gradient) followed by AddNode::backward (a sum over the
// batch) without the transposed copy. A workgroup owns 64 pixels x 32 channels: it starts from the values
// already in dbias and adds the images in ascending order (the order of the two-step chain), reading dz
// along pixels and writing dbias along channels; the tile is turned in LDS on the way in and on the way out.
// MASK: dz is not given but made here, dz[n][o][p] = y[n][o][p] > 0 ? dy[n][o][p] : 0 (the gradient through the ReLU
// that follows the convolution, ReLUNode::backward), written out for the other gradient kernels and summed on the way.
template <bool MASK>
__global__ __launch_bounds__(256) void conv_bias_grad_kernel(float* __restrict__ dbias, const float* __restrict__ dz, int N,
                                                             int O, long HW, float* __restrict__ dz_out,
                                                             const float* __restrict__ y) {
    __shared__ float tile[64][33];                               // [pixel][channel]
    const long p0 = (long)blockIdx.x * 64;
    const int o0 = blockIdx.y * 32;
    {   // in: rows of dbias (channels contiguous)
        const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
#pragma unroll
        for (int r = 0; r < 64; r += 8) {
            const long p = p0 + ty + r;
            const int o = o0 + tx;
            tile[ty + r][tx] = (p < HW && o < O) ? dbias[p * O + o] : 0.f;
        }
    }
    __syncthreads();
    const int px = threadIdx.x & 63, oy = threadIdx.x >> 6;      // this thread's pixel, and channels oy, oy + 4, ...
    const long p = p0 + px;
    float acc[8];
#pragma unroll
    for (int r = 0; r < 8; r++) acc[r] = tile[px][oy + r * 4];
    if (p < HW)
        for (int n = 0; n < N; n++) {
#pragma unroll
            for (int r = 0; r < 8; r++) {
                const int o = o0 + oy + r * 4;
                if (o < O) {
                    const long at = ((long)n * O + o) * HW + p;
                    float g = dz[at];
                    if (MASK) {
                        g = y[at] > 0.f ? g : 0.f;
                        dz_out[at] = g;
                    }
                    acc[r] += g;
                }
            }
        }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 8; r++) tile[px][oy + r * 4] = acc[r];
    __syncthreads();
    {   // out: rows of dbias again
        const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
#pragma unroll
        for (int r = 0; r < 64; r += 8) {
            const long pp = p0 + ty + r;
            const int o = o0 + tx;
            if (pp < HW && o < O) dbias[pp * O + o] = tile[ty + r][tx];
        }
    }
}

// Weights of the data-gradient convolution: the gradient with respect to x of a stride-1 convolution is
// itself a stride-1 convolution of dy (O channels in, C channels out) with the taps mirrored:
//   w'[wb][(o, r', s')][c] = w[wb][(c, K_h-1-r', K_w-1-s')][o]
__global__ __launch_bounds__(256) void conv_weight_flip_kernel(float* __restrict__ dst, const float* __restrict__ src,
                                                               int C, int O, int K_h, int K_w, long total) {
    const long t = (long)blockIdx.x * 256 + threadIdx.x;      // index into dst, c fastest
    if (t >= total) return;
    const int taps = K_h * K_w;
    const int c = (int)(t % C);
    const long q = t / C;                                       // (wb, o, r', s')
    const int tap = (int)(q % taps), o = (int)((q / taps) % O);
    const long wb = q / ((long)taps * O);
    const int r = K_h - 1 - tap / K_w, sx = K_w - 1 - tap % K_w;
    dst[t] = src[((wb * C + c) * taps + (long)r * K_w + sx) * O + o];
}

__global__ __launch_bounds__(256) void accumulate_kernel(float* __restrict__ dst, const float* __restrict__ src, long n) {
    const long t = ((long)blockIdx.x * 256 + threadIdx.x) * 4;
    if (t + 4 <= n && ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15) == 0) {
        floatx4 a = *reinterpret_cast<const floatx4*>(dst + t), b = *reinterpret_cast<const floatx4*>(src + t);
        a[0] += b[0]; a[1] += b[1]; a[2] += b[2]; a[3] += b[3];
        *reinterpret_cast<floatx4*>(dst + t) = a;
    } else {
        for (long i = t; i < n && i < t + 4; i++) dst[i] += src[i];
    }
}

}  // namespace nzhip

namespace nzhip {
// A 1x1 convolution with a stride and no padding only ever looks at every stride-th pixel of every stride-th row:
// dst[plane][ho][wo] = src[plane][ho * stride][wo * stride]. On that smaller image it is the 1x1 stride-1 convolution,
// forward and both gradients (the reference lowers it like any other: column matrix, product, and for the data
// gradient a scatter over the windows, src/Nodes.cu:605-640).
// A workgroup takes 256 >> wq_log rows of 1 << wq_log threads, a thread four adjacent columns of its row (one 16-byte
// store when the rows allow it): one division per thread instead of three per element.
template <bool VEC>
__global__ __launch_bounds__(256) void subsample_kernel(float* __restrict__ dst, const float* __restrict__ src, long rows, int H, int W,
                                                        int Ho, int Wo, int stride, int wq_log) {
    const long row = (long)blockIdx.x * (256 >> wq_log) + (threadIdx.x >> wq_log);      // (plane, ho)
    if (row >= rows) return;
    const long plane = rows <= 0x7fffffffl ? (long)((unsigned)row / (unsigned)Ho) : row / Ho;
    const int ho = (int)(row - plane * Ho);
    const float* srow = src + (plane * H + (long)ho * stride) * W;
    float* drow = dst + row * Wo;
    for (int w0 = (threadIdx.x & ((1 << wq_log) - 1)) * 4; w0 < Wo; w0 += 4 << wq_log) {
        floatx4 v;
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = srow[(long)min(w0 + j, Wo - 1) * stride];
        if (VEC) {
            *reinterpret_cast<floatx4*>(drow + w0) = v;
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (w0 + j < Wo) drow[w0 + j] = v[j];
        }
    }
}
// The way back: dst[plane][h][w] (+)= src[plane][h / stride][w / stride] where both divide and the source pixel exists;
// the other pixels get nothing (zero when dst is overwritten). The data gradient of a strided 1x1 convolution put back
// between the pixels it never looked at, and the output gradient of any strided convolution spread out to the positions
// its windows started at. Same thread layout as above; rows that no source row reaches are one store per piece (or
// nothing at all when accumulating).
template <bool VEC>
__global__ __launch_bounds__(256) void spread_strided_kernel(float* __restrict__ dst, const float* __restrict__ src, long rows, int H, int W,
                                                             int Ho, int Wo, int stride, int accumulate, int wq_log) {
    const long row = (long)blockIdx.x * (256 >> wq_log) + (threadIdx.x >> wq_log);      // (plane, h)
    if (row >= rows) return;
    const long plane = rows <= 0x7fffffffl ? (long)((unsigned)row / (unsigned)H) : row / H;
    const int h = (int)(row - plane * H);
    const int ho = h / stride;
    const bool row_hit = ho * stride == h && ho < Ho;
    if (accumulate && !row_hit) return;
    const float* srow = src + (plane * Ho + (row_hit ? ho : 0)) * Wo;
    float* drow = dst + row * W;
    for (int w0 = (threadIdx.x & ((1 << wq_log) - 1)) * 4; w0 < W; w0 += 4 << wq_log) {
        int wo = (w0 + stride - 1) / stride;          // the first source column at or right of w0
        int w_next = wo * stride;
        floatx4 v;
        bool hits[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            hits[j] = row_hit && w0 + j == w_next && wo < Wo;
            v[j] = hits[j] ? srow[wo] : 0.f;
            if (w0 + j == w_next) { w_next += stride; wo++; }
        }
        if (VEC) {
            if (accumulate) {                           // pixels without a source keep their bits
                const floatx4 old = *reinterpret_cast<const floatx4*>(drow + w0);
#pragma unroll
                for (int j = 0; j < 4; j++) v[j] = hits[j] ? old[j] + v[j] : old[j];
            }
            *reinterpret_cast<floatx4*>(drow + w0) = v;
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (w0 + j < W && (hits[j] || !accumulate)) drow[w0 + j] = accumulate ? drow[w0 + j] + v[j] : v[j];
        }
    }
}
// log2 of the threads per row: the power of two that covers a row's 4-column pieces, 256 at most
static int strided_wq_log(size_t W) {
    int l = 0;
    while (l < 8 && ((size_t)4 << l) < W) l++;
    return l;
}
static int spread_strided(float* dst, const float* src, size_t planes, size_t H, size_t W, size_t Ho, size_t Wo, size_t stride,
                          int accumulate, hipStream_t s) {
    const size_t rows = planes * H;
    const int wq_log = strided_wq_log(W);
    const size_t blocks = (rows + (256 >> wq_log) - 1) / (256 >> wq_log);
    if (H > 0x3fffffff || W > 0x3fffffff || blocks > 0x7fffffffull)
        return set_error(NZHIP_E_UNSUPPORTED, "nzhip_conv2d_backward_data: extents beyond the fused kernels (use the column-matrix chain)");
    if (rows == 0 || W == 0) return NZHIP_OK;
    const bool vec = W % 4 == 0 && (reinterpret_cast<uintptr_t>(dst) & 15) == 0;
    hipLaunchKernelGGL(vec ? spread_strided_kernel<true> : spread_strided_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, s, dst, src,
                       (long)rows, (int)H, (int)W, (int)Ho, (int)Wo, (int)stride, accumulate, wq_log);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? NZHIP_OK : set_hip_error(e, "spread_strided kernel launch");
}
static bool conv1x1_strided(size_t K_h, size_t K_w, size_t stride, size_t pad, size_t N, size_t C, size_t H, size_t W) {
    return K_h == 1 && K_w == 1 && stride > 1 && pad == 0 && H > 0 && W > 0 && H < 0x3fffffff && W < 0x3fffffff &&
           (N * C * H * W + 255) / 256 < 0x7fffffffull;
}
// x [N, C, H, W] -> a pooled workspace [N, C, Ho, Wo] with every stride-th pixel of every stride-th row
static int conv_subsample(float** sub, const float* x, size_t planes, size_t H, size_t W, size_t Ho, size_t Wo, size_t stride, hipStream_t s) {
    const size_t total = planes * Ho * Wo;
    if (int rc = workspace_alloc(reinterpret_cast<void**>(sub), total * sizeof(float), s)) return rc;
    const size_t rows = planes * Ho;
    const int wq_log = strided_wq_log(Wo);
    const bool vec = Wo % 4 == 0;                       // pooled workspaces are 256-byte aligned
    hipLaunchKernelGGL(vec ? subsample_kernel<true> : subsample_kernel<false>, dim3((unsigned)((rows + (256 >> wq_log) - 1) / (256 >> wq_log))),
                       dim3(256), 0, s, *sub, x, (long)rows, (int)H, (int)W, (int)Ho, (int)Wo, (int)stride, wq_log);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        workspace_free(*sub, s);
        return set_hip_error(e, "subsample kernel launch");
    }
    return NZHIP_OK;
}
}  // namespace nzhip

using namespace nzhip;

// bias_stride_image != 0: the bias varies per image too (used to add into an existing tensor: bias = y with
// strides (1, H_out*W_out, O*H_out*W_out)); only the implicit-GEMM kernels take it.
// Which kernel family a forward convolution takes (a per-image bias, which only the data gradient uses, does not change
// the choice; the two implicit-GEMM families support it, the others do not).
enum ConvRoute { CONV_ROUTE_DIRECT, CONV_ROUTE_FIXED, CONV_ROUTE_ANY, CONV_ROUTE_WORKSPACE };

static ConvRoute conv_forward_route(const float* x, size_t N, size_t C, size_t H, size_t W, size_t O, size_t K_h, size_t K_w, size_t stride,
                                    size_t pad, size_t w_batch, size_t H_out, size_t W_out, bool& wide, bool& bn128) {
    static const char* route_env = getenv("NZHIP_CONV_ROUTE");      // "workspace": column matrix + GEMM; "gen": the any-geometry
                                                                     // kernel wherever it applies (benchmarking only)
    // NZHIP_CONV_TW=32|64 and NZHIP_CONV_BN=64|128 override the tile choice (benchmarking only)
    static const char* tw_env = getenv("NZHIP_CONV_TW");
    static const char* bn_env = getenv("NZHIP_CONV_BN");
    wide = tw_env ? atoi(tw_env) == 64 : W_out >= 64;
    bn128 = bn_env ? atoi(bn_env) == 128 : O > 64;
    if (conv_direct_applicable(C, O, K_h, K_w, stride, pad)) return CONV_ROUTE_DIRECT;
    const bool force_ws = route_env && route_env[0] == 'w', force_gen = route_env && route_env[0] == 'g';
    if (force_ws) return CONV_ROUTE_WORKSPACE;
    // One weight copy per image, each used for a single small image: the fp16 image the implicit-GEMM kernels want costs a
    // pass over all copies (read fp32, write fp16, read fp16 again) for weights the column-matrix product reads once as they
    // lie. Cheaper whenever the column matrix is smaller than the weights, output pixels x 2 <= output channels
    // (16 x 512 x 14 x 14 -> 512, 151 MB of weights: 103 against 130 us; the data gradient 83 against 133), unless the caller
    // keeps the image across calls.
    if (w_batch > 1 && !force_gen && K_h * K_w > 1 && H_out * W_out * 2 <= O && !image_kept_by_caller(PREPARED_CONV_W))
        return CONV_ROUTE_WORKSPACE;
    const bool fixed_ok = conv_igemm_applicable(C, O, K_h, K_w, stride, pad, N) && (long)H * W < 0x7fffffffL;
    // Small images with many channels: the weights do not fit LDS, so the implicit-GEMM kernel runs one
    // patch per workgroup with the whole C x taps contraction inside, and there are too few patches to
    // fill the CUs (8 x 512 x 16 x 16 -> 512: 64 workgroups, 190 us). The column matrix of such a layer is
    // small; its batched GEMM splits the contraction over the idle CUs instead (83 us).
    bool few_patches = false, sparse_patches = false, long_contraction = false;
    {
        const size_t tw = wide ? 64 : 32, th = 256 / tw, bn = bn128 ? 128 : 64;
        const size_t units = N * ((W_out + tw - 1) / tw) * ((H_out + th - 1) / th) * ((O + bn - 1) / bn);
        const size_t w_lds = ((C + IG_CC - 1) / IG_CC) * bn * K_h * K_w * 32;       // fp16 weight image of one channel tile
        const bool resident = (w_batch == 1 || N * ((O + bn - 1) / bn) <= (size_t)device_cu_count()) && w_lds <= 148 * 1024;
        few_patches = !resident && units * 4 <= (size_t)device_cu_count();
        // Weights beyond LDS and fewer than 1.75 patches per compute unit (16 x 256 x 28 x 28 -> 256: 128): the any-geometry
        // kernel splits the channels over workgroups and is faster there (58 against 87 us; 16 x 512 x 16 x 16 -> 512: 75
        // against 193 us), as long as its 256-pixel segments are at least half full (4 x 512 x 8 x 8: 37 against 29 us).
        sparse_patches = !resident && units * 4 < 7 * (size_t)device_cu_count();
        // Weights beyond LDS and 192 or more input channels: the any-geometry kernel takes two chunks per step there and is
        // 3-8 % faster than one patch per workgroup (16 x 512 x 28 x 28 -> 512: 118 against 128 us; 16 x 192 x 64 x 64 -> 192:
        // 82 against 87; with 128 channels the two are level or the other way round)
        long_contraction = !resident && C >= 192 && K_h == 3 && K_w == 3 && W % 4 == 0;
    }
    // any other kernel extent or stride, when the segments (times the channel groups the contraction can be split into)
    // occupy at least a quarter of the CUs
    if ((!fixed_ok || force_gen || sparse_patches || long_contraction) && conv_igemm_gen_applicable(x, C, H, W, O, K_h, K_w, stride, pad, N) &&
        (w_batch == 1 || w_batch * ((O + 63) / 64) * ((C + 15) / 16) <= 65535) && conv_igemm_gen_fits(W_out, O, K_h, K_w, stride, pad)) {
        const int sw_log = conv_igemm_gen_sw_log(W_out, O, K_h, K_w, stride, pad);     // (not 0: it fits)
        const size_t sw = (size_t)1 << sw_log, sr = CG_PX / sw;
        const size_t chunks = (C + IG_CC - 1) / IG_CC;
        const size_t seg_rows = (H_out + sr - 1) / sr, segs_w = (W_out + sw - 1) / sw;
        const size_t groups = N * seg_rows * segs_w * ((O + 127) / 128) * (chunks >= 4 ? chunks / 2 : 1);
        const bool half_full = H_out * W_out * 2 >= seg_rows * sr * segs_w * sw;
        // (segments less than half full -- 7 x 7 or 8 x 8 outputs in 16 x 16 pixel segments -- multiply mostly padding:
        // 16 x 512 x 14 x 14 -> 512 at stride 2 116 us here, 47 us through the column matrix)
        if (force_gen || (groups * 4 >= (size_t)device_cu_count() && half_full)) return CONV_ROUTE_ANY;
    }
    return fixed_ok && !few_patches ? CONV_ROUTE_FIXED : CONV_ROUTE_WORKSPACE;
}

// w_mirror: w_ref is the parameter of the convolution whose DATA GRADIENT this call computes ([(c_f, tap)][o_f] with
// c_f running over this call's O channels and o_f over its C), to be used with channels swapped and taps mirrored.
// The implicit-GEMM routes read it that way while they build their fp16 weight image; the routes that take the
// weights as they lie (column matrix, direct kernels) get a mirrored copy first.
static int conv2d_forward_impl(float* y, const float* x, const float* w_ref, const float* bias, size_t N, size_t C,
                               size_t H, size_t W, size_t O, size_t K_h, size_t K_w, size_t stride, size_t pad,
                               size_t w_batch, int64_t bias_stride_pixel, int64_t bias_stride_channel,
                               int64_t bias_stride_image, int activation, void* stream, bool w_mirror = false);
static int conv2d_forward_mirrored_copy(float* y, const float* x, const float* w_ref, const float* bias, size_t N, size_t C,
                                        size_t H, size_t W, size_t O, size_t K_h, size_t K_w, size_t stride, size_t pad,
                                        size_t w_batch, int64_t bias_stride_pixel, int64_t bias_stride_channel,
                                        int64_t bias_stride_image, int activation, void* stream) {
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const size_t w_elems = w_batch * C * K_h * K_w * O;
    float* wflip = nullptr;
    if (int rc = workspace_alloc(reinterpret_cast<void**>(&wflip), w_elems * sizeof(float), s)) return rc;
    // the copy is this call's own parameter: [(c, tap)][o] with c over this call's C input channels
    hipLaunchKernelGGL(conv_weight_flip_kernel, dim3((unsigned)((w_elems + 255) / 256)), dim3(256), 0, s, wflip, w_ref, (int)O, (int)C,
                       (int)K_h, (int)K_w, (long)w_elems);
    hipError_t e = hipGetLastError();
    int rc = e == hipSuccess ? NZHIP_OK : set_hip_error(e, "conv_weight_flip kernel launch");
    if (rc == NZHIP_OK)
        rc = conv2d_forward_impl(y, x, wflip, bias, N, C, H, W, O, K_h, K_w, stride, pad, w_batch, bias_stride_pixel,
                                 bias_stride_channel, bias_stride_image, activation, stream, false);
    const int rc2 = workspace_free(wflip, s);
    return rc ? rc : rc2;
}
static int conv2d_forward_impl(float* y, const float* x, const float* w_ref, const float* bias, size_t N, size_t C,
                               size_t H, size_t W, size_t O, size_t K_h, size_t K_w, size_t stride, size_t pad,
                               size_t w_batch, int64_t bias_stride_pixel, int64_t bias_stride_channel,
                               int64_t bias_stride_image, int activation, void* stream, bool w_mirror) {
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
    if (w_mirror && (K_h != K_w || (K_h == 1 && K_w == 1)))     // mirrored taps as one reversed index need a square kernel; 1x1 routes take the weights as they lie
        return conv2d_forward_mirrored_copy(y, x, w_ref, bias, N, C, H, W, O, K_h, K_w, stride, pad, w_batch, bias_stride_pixel,
                                            bias_stride_channel, bias_stride_image, activation, stream);
    if (conv1x1_strided(K_h, K_w, stride, pad, N, C, H, W) && H_out * W_out >= 64) {
        // 1x1 with a stride: gather the pixels it looks at, then the 1x1 stride-1 convolution of the smaller image
        // (16 x 512 x 28 x 28 -> 1024 at stride 2: 42 -> 32 us; not with fewer than 64 pixels left per image, where the
        // column matrix and one product over all images is the better way: 16 x 1024 x 14 x 14 -> 2048: 39 against 72 us)
        float* sub = nullptr;
        if (int rc = conv_subsample(&sub, x, N * C, H, W, H_out, W_out, stride, s)) return rc;
        const int rc = conv2d_forward_impl(y, sub, w_ref, bias, N, C, H_out, W_out, O, 1, 1, 1, 0, w_batch, bias_stride_pixel,
                                           bias_stride_channel, bias_stride_image, activation, stream);
        const int rc2 = workspace_free(sub, s);
        return rc ? rc : rc2;
    }
    // 1x1, stride 1, no padding: no window at all, y[n] (O x pixels) = W^T (O x C) * x[n] (C x pixels) is one batched product,
    // every bias form is a bias matrix with strides. From 32 input channels on that is level with or ahead of the implicit-GEMM
    // kernels (16 x 64 x 56 x 56 -> 64: 12 against 18 us; 16 x 120 x 56 x 56 -> 120 with the reference's per-pixel bias: 23 against
    // 30 us), and with at least 128 well ahead
    // (16 x 512 x 28 x 28 -> 128: 16 against 31 us; 16 x 256 x 14 x 14 -> 1024: 20 against 55 us), tiny images included since
    // their planes are widened to whole 16-byte pieces (16 x 512 x 7 x 7 -> 128: 14 against 47 us through the column matrix).
    static const char* gemm1x1_env = getenv("NZHIP_CONV_1X1_GEMM");     // benchmarking only: 0 never, 1 always
    const bool as_product = K_h == 1 && K_w == 1 && stride == 1 && pad == 0 && H * W < 0x3fffffff && C < 0x3fffffff && O < 0x3fffffff &&
                            N <= 65535 &&
                            (gemm1x1_env ? atoi(gemm1x1_env) != 0 : C >= 32);
    if (as_product) {
        nzhip_gemm_desc g = {};
        g.A = w_ref; g.M = (int64_t)O; g.K = (int64_t)C; g.lda = (int64_t)O; g.a_layout = NZHIP_LAYOUT_TRANS;   // w_ref holds C x O
        g.B = x; g.N = (int64_t)(H * W); g.ldb = (int64_t)(H * W); g.b_layout = NZHIP_LAYOUT_ROW;
        g.C = y; g.ldc = (int64_t)(H * W);
        g.batch_n = (int64_t)N; g.batch_c = 1;
        g.a_stride_n = w_batch > 1 ? (int64_t)(C * O) : 0; g.b_stride_n = (int64_t)(C * H * W); g.c_stride_n = (int64_t)(O * H * W);
        g.bias = bias; g.bias_stride_row = bias_stride_channel; g.bias_stride_col = bias_stride_pixel; g.bias_stride_n = bias_stride_image;
        g.activation = activation;
        // The reference's bias is pixel-major ([1, 1, pixels, O], src/Model.cu:252-256) while the product's lanes run along
        // the pixels: read as it lies, every bias load touches 64 lines 4 O bytes apart. One pass turns it into channel
        // planes, the layout of y (16 x 64 x 56 x 56 -> 256: 41 -> 33 us).
        float* bias_planes = nullptr;
        if (bias && bias_stride_image == 0 && bias_stride_channel == 1 && bias_stride_pixel == (int64_t)O && O >= 8 && O * H * W >= 262144) {      // from 1 MB of bias on: below, the pass costs what it saves
            if (int rc = workspace_alloc(reinterpret_cast<void**>(&bias_planes), O * H * W * sizeof(float), s)) return rc;
            if (int rc = nzhip_col2im(bias_planes, bias, H, W, O, 1, s)) {
                workspace_free(bias_planes, s);
                return rc;
            }
            g.bias = bias_planes; g.bias_stride_row = (int64_t)(H * W); g.bias_stride_col = 1;
        }
        float* x_wide = nullptr;
        const double flops = 2.0 * (double)N * (double)(H * W) * (double)C * (double)O;
        if (conv1x1_wants_wide_planes(H * W, flops, 2.0 * (double)O)) {
            if (int rc = widen_rows(&x_wide, x, N * C, H * W, s)) {
                if (bias_planes) workspace_free(bias_planes, s);
                return rc;
            }
            const size_t HWp = (H * W + 3) / 4 * 4;
            g.B = x_wide; g.ldb = (int64_t)HWp; g.b_stride_n = (int64_t)(C * HWp);
        }
        const int rc = x_wide ? gemm_padded_rows(g, 2, s) : nzhip_gemm(&g, s);
        const int rc2 = x_wide ? workspace_free(x_wide, s) : NZHIP_OK;
        const int rc3 = bias_planes ? workspace_free(bias_planes, s) : NZHIP_OK;
        return rc ? rc : (rc2 ? rc2 : rc3);
    }
    bool wide = false, bn128 = false;
    const ConvRoute route = conv_forward_route(x, N, C, H, W, O, K_h, K_w, stride, pad, w_batch, H_out, W_out, wide, bn128);
    const bool fixed_geometry = route == CONV_ROUTE_FIXED, any_geometry = route == CONV_ROUTE_ANY;
    if (bias_stride_image != 0 && !fixed_geometry && !any_geometry)
        return set_error(NZHIP_E_UNSUPPORTED, "conv2d: a per-image bias needs an implicit-GEMM route");
    if (w_mirror && !fixed_geometry && !any_geometry)
        return conv2d_forward_mirrored_copy(y, x, w_ref, bias, N, C, H, W, O, K_h, K_w, stride, pad, w_batch, bias_stride_pixel,
                                            bias_stride_channel, bias_stride_image, activation, stream);
    if (route == CONV_ROUTE_DIRECT)
        return conv_direct(y, x, w_ref, bias, N, C, H, W, O, w_batch, bias_stride_pixel, bias_stride_channel,
                           activation, s);
    if (fixed_geometry || any_geometry) {
        // The reference's bias parameter is pixel-major ([1,1,H_out*W_out,O], src/Model.cu:252-256), while the kernels'
        // lanes are adjacent pixels: read as it lies, every bias load touches 64 lines 4 O bytes apart. One pass turns it
        // into channel planes (the layout of y), and the bias loads look like the result stores.
        const float* bias_use = bias;
        int64_t bsp = bias_stride_pixel, bsc = bias_stride_channel;
        float* bias_planes = nullptr;
        if (bias && bias_stride_image == 0 && bsc == 1 && bsp == (int64_t)O && O >= 8 && H_out * W_out >= 64) {
            if (int rc = workspace_alloc(reinterpret_cast<void**>(&bias_planes), O * H_out * W_out * sizeof(float), s)) return rc;
            if (int rc = nzhip_col2im(bias_planes, bias, H_out, W_out, O, 1, s)) {
                workspace_free(bias_planes, s);
                return rc;
            }
            bias_use = bias_planes; bsp = 1; bsc = (int64_t)(H_out * W_out);
        }
        auto finish = [&](int rc) {
            const int rc2 = bias_planes ? workspace_free(bias_planes, s) : NZHIP_OK;
            return rc ? rc : rc2;
        };
        if (any_geometry) {
            const int rc = conv_igemm_gen_launch(y, x, w_ref, bias_use, N, C, H, W, O, K_h, K_w, stride, pad, w_batch, bsp, bsc,
                                                 bias_stride_image, activation, H_out, W_out, w_mirror, s);
            const int rc_free = finish(rc == NZHIP_E_UNSUPPORTED ? NZHIP_OK : rc);
            if (rc != NZHIP_E_UNSUPPORTED) return rc_free;
            if (bias_stride_image != 0) return set_error(NZHIP_E_UNSUPPORTED, "conv2d: a per-image bias needs an implicit-GEMM route");
            if (w_mirror) {                                                                   // the column-matrix route needs the weights as they lie
                float* wflip = nullptr;
                const size_t w_elems = w_batch * C * K_h * K_w * O;
                if (int rc_a = workspace_alloc(reinterpret_cast<void**>(&wflip), w_elems * sizeof(float), s)) return rc_a;
                hipLaunchKernelGGL(conv_weight_flip_kernel, dim3((unsigned)((w_elems + 255) / 256)), dim3(256), 0, s, wflip, w_ref, (int)O,
                                   (int)C, (int)K_h, (int)K_w, (long)w_elems);
                hipError_t e = hipGetLastError();
                int rc_w = e == hipSuccess ? NZHIP_OK : set_hip_error(e, "conv_weight_flip kernel launch");
                if (rc_w == NZHIP_OK)
                    rc_w = conv2d_via_workspace(y, x, wflip, bias, N, C, H, W, O, K_h, K_w, stride, pad, w_batch, bias_stride_pixel,
                                                bias_stride_channel, activation, H_out, W_out, s);
                const int rc_f = workspace_free(wflip, s);
                return rc_w ? rc_w : rc_f;
            }
            return conv2d_via_workspace(y, x, w_ref, bias, N, C, H, W, O, K_h, K_w, stride, pad, w_batch, bias_stride_pixel,
                                        bias_stride_channel, activation, H_out, W_out, s);   // the tile does not fit: column matrix
        }
#define NZHIP_IG(KH_, TW_, BN_)                                                                                      \
    return finish(conv_igemm_launch<KH_, KH_, TW_, BN_>(y, x, w_ref, bias_use, N, C, H, W, O, pad, w_batch, bsp, bsc, \
                                                        bias_stride_image, activation, H_out, W_out, w_mirror, s))
        if (K_h == 3) {
            if (wide && bn128) NZHIP_IG(3, 64, 128);
            if (wide) NZHIP_IG(3, 64, 64);
            if (bn128) NZHIP_IG(3, 32, 128);
            NZHIP_IG(3, 32, 64);
        }
        if (wide) NZHIP_IG(1, 64, 64);
        NZHIP_IG(1, 32, 64);
#undef NZHIP_IG
    }
    return conv2d_via_workspace(y, x, w_ref, bias, N, C, H, W, O, K_h, K_w, stride, pad, w_batch, bias_stride_pixel,
                                bias_stride_channel, activation, H_out, W_out, s);
}

extern "C" int nzhip_conv2d_forward(float* y, const float* x, const float* w_ref, const float* bias, size_t N,
                                    size_t C, size_t H, size_t W, size_t O, size_t K_h, size_t K_w, size_t stride,
                                    size_t pad, size_t w_batch, int64_t bias_stride_pixel,
                                    int64_t bias_stride_channel, int activation, void* stream) {
    return conv2d_forward_impl(y, x, w_ref, bias, N, C, H, W, O, K_h, K_w, stride, pad, w_batch, bias_stride_pixel,
                               bias_stride_channel, 0, activation, stream);
}

namespace nzhip {
// img2colBackwardKernel (src/OperationKernels.cu:1337-1355) as a gather from the TRANSPOSED column gradient
// colT[image][(c, r, s)][pixel] (rows `pitch` floats apart): one thread owns one element of dx and adds the entries that
// were copied from it in ascending pixel order, the order of the library's im2col_backward kernel and of the reference's
// element index. With the pixels contiguous, the threads of a wave (adjacent w) read adjacent addresses; from the
// reference's layout [pixel][(c, r, s)] every lane touches a line of its own.
__global__ __launch_bounds__(256) void col_t_gather_kernel(float* __restrict__ dx, const float* __restrict__ colT, int H_out, int W_out,
                                                           int C, int K_h, int K_w, int stride, int pad, int H_in, int W_in, long pitch,
                                                           int accumulate) {
    const long per_img = (long)C * H_in * W_in;
    const long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= per_img) return;
    const int b = blockIdx.y;
    const int c = (int)(t / ((long)H_in * W_in));
    const int h = (int)((t / W_in) % H_in), w = (int)(t % W_in);
    const float* col = colT + ((long)b * C + c) * K_h * K_w * pitch;
    float acc = accumulate ? dx[(long)b * per_img + t] : 0.f;
    const int ho_lo = h + pad - K_h + 1 > 0 ? (h + pad - K_h + 1 + stride - 1) / stride : 0;
    const int ho_hi = (h + pad) / stride < H_out - 1 ? (h + pad) / stride : H_out - 1;
    const int wo_lo = w + pad - K_w + 1 > 0 ? (w + pad - K_w + 1 + stride - 1) / stride : 0;
    const int wo_hi = (w + pad) / stride < W_out - 1 ? (w + pad) / stride : W_out - 1;
    for (int ho = ho_lo; ho <= ho_hi; ho++) {
        const int r = h + pad - ho * stride;
        for (int wo = wo_lo; wo <= wo_hi; wo++) {
            const int sx = w + pad - wo * stride;
            acc += col[(long)(r * K_w + sx) * pitch + (long)ho * W_out + wo];
        }
    }
    dx[(long)b * per_img + t] = acc;
}
}  // namespace nzhip

// The reference's own chain for the data gradient (src/Nodes.cu:660-665, 169-182, 632-640) inside the library, with the
// column gradient transposed: per image colT[(c, r, s)][pixel] = W [(c, r, s)][o] x dy[o][pixel] is a product on dy as
// it lies (no pixel-major copy of dy, no mirrored weights), and the gather into the image reads it along the pixels.
// Every entry is the same sum over o as in the reference's dC x B^T, and they are added into dx in the same order.
static int conv_dx_chain_planes(float* dx, const float* dy, const float* w_ref, size_t N, size_t C, size_t H, size_t W, size_t O, size_t K_h,
                                size_t K_w, size_t stride, size_t pad, size_t Ho, size_t Wo, size_t w_batch, int accumulate, void* stream) {
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const size_t P = Ho * Wo, Pp = (P + 3) / 4 * 4, CKK = C * K_h * K_w;
    if ((C * H * W + 255) / 256 > 0x7fffffffull) return set_error(NZHIP_E_UNSUPPORTED, "nzhip_conv2d_backward_data: image beyond the gather kernel's grid");
    float* colT = nullptr;
    float* dy_wide = nullptr;
    if (int rc = workspace_alloc(reinterpret_cast<void**>(&colT), N * CKK * Pp * sizeof(float), s)) return rc;
    int rc = NZHIP_OK;
    if (P % 4 != 0) rc = widen_rows(&dy_wide, dy, N * O, P, s);       // planes of whole 16-byte pieces for the product's loads
    if (rc == NZHIP_OK) {
        nzhip_gemm_desc g = {};
        g.A = w_ref; g.M = (int64_t)CKK; g.K = (int64_t)O; g.lda = (int64_t)O; g.a_layout = NZHIP_LAYOUT_ROW;   // w_ref holds CKK x O
        g.B = dy_wide ? dy_wide : dy; g.N = (int64_t)P; g.ldb = (int64_t)(dy_wide ? Pp : P); g.b_layout = NZHIP_LAYOUT_ROW;
        g.C = colT; g.ldc = (int64_t)Pp;
        g.batch_n = (int64_t)N; g.batch_c = 1;
        g.a_stride_n = w_batch > 1 ? (int64_t)(CKK * O) : 0; g.b_stride_n = (int64_t)(O * (dy_wide ? Pp : P)); g.c_stride_n = (int64_t)(CKK * Pp);
        g.activation = NZHIP_ACT_NONE;
        rc = dy_wide ? gemm_padded_rows(g, 2, s) : nzhip_gemm(&g, s);
    }
    if (rc == NZHIP_OK) {
        hipLaunchKernelGGL(col_t_gather_kernel, dim3((unsigned)((C * H * W + 255) / 256), (unsigned)N), dim3(256), 0, s, dx, colT, (int)Ho,
                           (int)Wo, (int)C, (int)K_h, (int)K_w, (int)stride, (int)pad, (int)H, (int)W, (long)Pp, accumulate ? 1 : 0);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) rc = set_hip_error(e, "col_t_gather kernel launch");
    }
    const int rc2 = dy_wide ? workspace_free(dy_wide, s) : NZHIP_OK;
    const int rc3 = workspace_free(colT, s);
    return rc ? rc : (rc2 ? rc2 : rc3);
}

// The reference's own chain for the data gradient (src/Nodes.cu:660-665, 169-182, 632-640) inside the library, in the
// reference's layouts: the output gradient pixel-major, the column gradient = dy^T x W^T as ONE product with all images
// as its rows, then the gather into the image. For images of fewer than 64 output pixels with shared weights: a product
// per image would read the weights once per image for a handful of columns (16 x 512 x 7 x 7 <- 512: 40 against 52 us).
static int conv_dx_chain_rows(float* dx, const float* dy, const float* w_ref, size_t N, size_t C, size_t H, size_t W, size_t O, size_t K_h,
                         size_t K_w, size_t stride, size_t pad, size_t Ho, size_t Wo, size_t w_batch, int accumulate, void* stream) {
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const size_t P = Ho * Wo, CKK = C * K_h * K_w;
    float* dyt = nullptr;
    float* dcol = nullptr;
    if (int rc = workspace_alloc(reinterpret_cast<void**>(&dyt), N * P * O * sizeof(float), s)) return rc;
    if (int rc = workspace_alloc(reinterpret_cast<void**>(&dcol), N * P * CKK * sizeof(float), s)) {
        workspace_free(dyt, s);
        return rc;
    }
    int rc = nzhip_col2im_backward(dyt, dy, Ho, Wo, O, N, stream);                 // [N][P][O]
    if (rc == NZHIP_OK) {
        nzhip_gemm_desc g = {};
        g.A = dyt; g.K = (int64_t)O; g.lda = (int64_t)O; g.a_layout = NZHIP_LAYOUT_ROW;
        g.B = w_ref; g.N = (int64_t)CKK; g.ldb = (int64_t)O; g.b_layout = NZHIP_LAYOUT_TRANS;       // w_ref holds CKK x O
        g.C = dcol; g.ldc = (int64_t)CKK;
        g.batch_c = 1;
        if (w_batch > 1) {                                                           // one product per image
            g.M = (int64_t)P; g.batch_n = (int64_t)N;
            g.a_stride_n = (int64_t)(P * O); g.b_stride_n = (int64_t)(CKK * O); g.c_stride_n = (int64_t)(P * CKK);
        } else {                                                                     // all images as rows of one product
            g.M = (int64_t)(N * P); g.batch_n = 1;
        }
        g.activation = NZHIP_ACT_NONE;
        rc = nzhip_gemm(&g, s);
    }
    if (rc == NZHIP_OK && !accumulate) rc = nzhip_fill(dx, 0.f, N * C * H * W, stream);
    if (rc == NZHIP_OK) rc = nzhip_im2col_backward(dx, dcol, Ho, Wo, C, K_h, K_w, stride, pad, H, W, N, stream);
    const int rc2 = workspace_free(dcol, s), rc3 = workspace_free(dyt, s);
    return rc ? rc : (rc2 ? rc2 : rc3);
}

static int conv_dx_chain(float* dx, const float* dy, const float* w_ref, size_t N, size_t C, size_t H, size_t W, size_t O, size_t K_h,
                         size_t K_w, size_t stride, size_t pad, size_t Ho, size_t Wo, size_t w_batch, int accumulate, void* stream) {
    if (w_batch == 1 && Ho * Wo < 64)
        return conv_dx_chain_rows(dx, dy, w_ref, N, C, H, W, O, K_h, K_w, stride, pad, Ho, Wo, w_batch, accumulate, stream);
    return conv_dx_chain_planes(dx, dy, w_ref, N, C, H, W, O, K_h, K_w, stride, pad, Ho, Wo, w_batch, accumulate, stream);
}

/* Gradient of nzhip_conv2d_forward with respect to x: one convolution of dy with the
 * mirrored weights instead of the reference's chain Col2ImgNode::backward -> MatMulNode::backward
 * (dA += dC * B^T) -> Img2ColNode::backward (src/Nodes.cu:660-665, 169-182, 632-640), which writes and
 * re-reads a column-matrix gradient of K_h*K_w times the size of x. With a stride above 1 the output gradient is first
 * spread out with zeros between its pixels; the stride-1 convolution of that is the same sum. */
extern "C" int nzhip_conv2d_backward_data(float* dx, const float* dy, const float* w_ref, size_t N, size_t C, size_t H,
                                          size_t W, size_t O, size_t K_h, size_t K_w, size_t stride, size_t pad,
                                          size_t w_batch, int accumulate, void* stream) {
    if (!dx || !dy || !w_ref) return set_error(NZHIP_E_INVALID, "nzhip_conv2d_backward_data: null pointer");
    if (stride == 0 || K_h == 0 || K_w == 0)
        return set_error(NZHIP_E_INVALID, "nzhip_conv2d_backward_data: zero stride or kernel extent");
    if (w_batch != 1 && w_batch != N) return set_error(NZHIP_E_SHAPE, "Shapes are not broadcast compatible.");
    if (H + 2 * pad < K_h || W + 2 * pad < K_w)
        return set_error(NZHIP_E_SHAPE, "nzhip_conv2d_backward_data: kernel larger than the padded input");
    if (stride > 8 || K_h != K_w || pad > K_h - 1)
        return set_error(NZHIP_E_UNSUPPORTED,
                         "nzhip_conv2d_backward_data: only square kernels, pad <= K-1 and stride <= 8 (use the column-matrix chain)");
    if (N == 0 || O == 0 || C == 0) return NZHIP_OK;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (conv1x1_strided(K_h, K_w, stride, pad, N, C, H, W) && ((H - 1) / stride + 1) * ((W - 1) / stride + 1) >= 64) {
        // 1x1 with a stride: the gradient of the pixels the convolution looked at, as a 1x1 stride-1 problem on the
        // smaller image, then put back between pixels that get none (16 x 512 x 28 x 28 <- 1024 at stride 2: 62 -> 45 us;
        // with fewer than 64 pixels left per image the per-image products are too small: 16 x 1024 x 14 x 14 <- 2048: 66 -> 86)
        const size_t Ho = (H - 1) / stride + 1, Wo = (W - 1) / stride + 1;
        float* sub = nullptr;
        if (int rc = workspace_alloc(reinterpret_cast<void**>(&sub), N * C * Ho * Wo * sizeof(float), s)) return rc;
        int rc = nzhip_conv2d_backward_data(sub, dy, w_ref, N, C, Ho, Wo, O, 1, 1, 1, 0, w_batch, 0, stream);
        if (rc == NZHIP_OK) rc = spread_strided(dx, sub, N * C, H, W, Ho, Wo, stride, accumulate ? 1 : 0, s);
        const int rc2 = workspace_free(sub, s);
        return rc ? rc : rc2;
    }
    if (K_h == 1 && stride == 1 && pad == 0 && H * W < 0x3fffffff && C < 0x3fffffff && O < 0x3fffffff && N <= 65535) {
        // 1x1: no window at all, dx[n] (C x pixels) (+)= W (C x O) * dy[n] (O x pixels), one batched product
        // (16 x 256 x 14 x 14 <- 1024 channels: 38 us against 99 us through the convolution kernels)
        nzhip_gemm_desc g = {};
        g.A = w_ref; g.M = (int64_t)C; g.K = (int64_t)O; g.lda = (int64_t)O; g.a_layout = NZHIP_LAYOUT_ROW;
        g.B = dy; g.N = (int64_t)(H * W); g.ldb = (int64_t)(H * W); g.b_layout = NZHIP_LAYOUT_ROW;
        g.C = dx; g.ldc = (int64_t)(H * W);
        g.batch_n = (int64_t)N; g.batch_c = 1;
        g.a_stride_n = w_batch > 1 ? (int64_t)(C * O) : 0; g.b_stride_n = (int64_t)(O * H * W); g.c_stride_n = (int64_t)(C * H * W);
        g.activation = NZHIP_ACT_NONE;
        if (accumulate) {
            g.bias = dx; g.bias_stride_n = g.c_stride_n; g.bias_stride_row = g.ldc; g.bias_stride_col = 1;
        }
        float* dy_wide = nullptr;
        const double flops = 2.0 * (double)N * (double)(H * W) * (double)C * (double)O;
        if (conv1x1_wants_wide_planes(H * W, flops, 2.0 * (double)C)) {
            if (int rc = widen_rows(&dy_wide, dy, N * O, H * W, s)) return rc;
            const size_t HWp = (H * W + 3) / 4 * 4;
            g.B = dy_wide; g.ldb = (int64_t)HWp; g.b_stride_n = (int64_t)(O * HWp);
        }
        const int rc = dy_wide ? gemm_padded_rows(g, 2, s) : nzhip_gemm(&g, s);
        const int rc2 = dy_wide ? workspace_free(dy_wide, s) : NZHIP_OK;
        return rc ? rc : rc2;
    }
    if (stride > 1) {
        const size_t Ho = (H + 2 * pad - K_h) / stride + 1, Wo = (W + 2 * pad - K_w) / stride + 1;
        // The convolution of the zero-filled gradient does stride^2 times the multiply-adds; the reference's own chain
        // (src/Nodes.cu:660-665, 169-182, 632-640: column gradient = W x dy, then the gather into the image) does them
        // once but writes and reads the column gradient. Many channels on small images favour the chain (16 x 512 x 14 x 14
        // <- 512 at stride 2: 42 against 71 us; 16 x 192 x 17 x 17 <- 192: 19 against 51), few channels on large images the
        // convolution (16 x 64 x 128 x 128 <- 128: 88 against 163). The estimate, in us, from the rates measured for both
        // sides on thirteen layers: the convolution at 600 (resident weights) or 300 TFLOP/s, half again as slow when the
        // zero-filled rows are not whole 16-byte pieces, plus the zero-filled gradient at 5 TB/s and 15-25 us for its four
        // launches; the chain's product at 500 TFLOP/s plus the column gradient (written, then gathered) at 1.1 TB/s and
        // 10 us for its launches.
        static const char* dx_env = getenv("NZHIP_CONV_DX");              // benchmarking only: "chain" | "conv"
        const double flops = 2.0 * N * Ho * Wo * C * K_h * K_w * O;
        const bool resident = ((O + 15) / 16) * (C > 64 ? 128 : 64) * K_h * K_w * 32 <= 148 * 1024;
        const double hu = (double)(H + 2 * pad - K_h + 1), wu = (double)(W + 2 * pad - K_w + 1);
        const bool pieces = (W + 2 * pad - K_w + 1) % 4 == 0;
        // (the convolution's output channels are the C input channels here, in tiles of 64: with 3 of them it multiplies
        // mostly padding, 16 x 3 x 224 x 224 <- 64 at 7x7 stride 2: 605 against 99 us)
        const double tile_fill = (double)((C + 63) / 64 * 64) / (double)C;
        const double as_conv = stride * stride * flops * tile_fill * (pieces ? 1.0 : 1.5) / (resident ? 600e6 : 300e6) +
                               N * O * hu * wu * 4.0 / 5e6 + (pieces ? 15.0 : 25.0);
        const double as_chain = 10.0 + flops / 500e6 + (double)N * Ho * Wo * C * K_h * K_w * 4.0 / 1.1e6;
        const size_t P = Ho * Wo, CKK = C * K_h * K_w;
        const bool chain_fits = N * P < 0x3fffffff && CKK < 0x3fffffff && O < 0x3fffffff && N <= 65535 && P * O < 0x7fffffffull &&
                                N * P * CKK <= ((size_t)1 << 29);      // a column gradient of at most 2 GiB
        if (chain_fits && (dx_env && dx_env[0] ? dx_env[1] == 'h' : as_conv >= as_chain))
            return conv_dx_chain(dx, dy, w_ref, N, C, H, W, O, K_h, K_w, stride, pad, Ho, Wo, w_batch, accumulate, stream);
        const size_t Hu = H + 2 * pad - K_h + 1, Wu = W + 2 * pad - K_w + 1, total = N * O * Hu * Wu;
        if (Hu > 0x3fffffff || Wu > 0x3fffffff)
            return set_error(NZHIP_E_UNSUPPORTED, "nzhip_conv2d_backward_data: extents beyond the fused kernels (use the column-matrix chain)");
        float* up = nullptr;
        if (int rc = workspace_alloc(reinterpret_cast<void**>(&up), total * sizeof(float), s)) return rc;
        int rc = spread_strided(up, dy, N * O, Hu, Wu, Ho, Wo, stride, 0, s);
        if (rc == NZHIP_OK) rc = nzhip_conv2d_backward_data(dx, up, w_ref, N, C, H, W, O, K_h, K_w, 1, pad, w_batch, accumulate, stream);
        const int rc2 = workspace_free(up, s);
        return rc ? rc : rc2;
    }
    const size_t H_out = H + 2 * pad - K_h + 1, W_out = W + 2 * pad - K_w + 1;
    const size_t x_elems = N * C * H * W;
    float* tmp = nullptr;
    int rc = NZHIP_OK;
    // "+=": the implicit-GEMM kernels read dx as their bias (same lane reads, then writes each element); the other
    // routes go through a temporary and one add pass
    const size_t pad_t = K_h - 1 - pad;
    bool wide_unused = false, bn_unused = false;
    const ConvRoute route = conv_forward_route(dy, N, O, H_out, W_out, C, K_h, K_w, 1, pad_t, w_batch, H, W, wide_unused, bn_unused);
    {
        // Where the convolution itself would write dy's column matrix (tiny images: 7 x 7, 4 x 4), the chain is the shorter
        // way: no mirrored copy of the weights, no column matrix of dy, no second pass for "+=" (16 x 512 x 7 x 7 <- 512, 3x3:
        // 56 -> 33 us).
        static const char* dx_env = getenv("NZHIP_CONV_DX");              // benchmarking only: "chain" | "conv"
        const size_t P = H_out * W_out, CKK = C * K_h * K_w;
        const bool chain_fits = N * P < 0x3fffffff && CKK < 0x3fffffff && O < 0x3fffffff && N <= 65535 && P * O < 0x7fffffffull &&
                                N * P * CKK <= ((size_t)1 << 28);
        const bool column_route = route != CONV_ROUTE_FIXED && route != CONV_ROUTE_ANY && route != CONV_ROUTE_DIRECT;
        if (chain_fits && (dx_env && dx_env[0] ? dx_env[1] == 'h' : column_route))
            return conv_dx_chain(dx, dy, w_ref, N, C, H, W, O, K_h, K_w, 1, pad, H_out, W_out, w_batch, accumulate, stream);
    }
    const bool in_place = accumulate && (route == CONV_ROUTE_FIXED || route == CONV_ROUTE_ANY);
    if (accumulate && !in_place) rc = workspace_alloc(reinterpret_cast<void**>(&tmp), x_elems * sizeof(float), s);
    // the weights go in as they are: the implicit-GEMM routes mirror them while they build their fp16 image, the others
    // make a mirrored copy themselves
    if (rc == NZHIP_OK && in_place)
        rc = conv2d_forward_impl(dx, dy, w_ref, dx, N, O, H_out, W_out, C, K_h, K_w, 1, pad_t, w_batch, 1, (int64_t)(H * W),
                                 (int64_t)(C * H * W), NZHIP_ACT_NONE, stream, true);
    else if (rc == NZHIP_OK)
        rc = conv2d_forward_impl(accumulate ? tmp : dx, dy, w_ref, nullptr, N, O, H_out, W_out, C, K_h, K_w, 1, pad_t,
                                 w_batch, 0, 0, 0, NZHIP_ACT_NONE, stream, true);
    if (rc == NZHIP_OK && accumulate && !in_place) {
        hipLaunchKernelGGL(accumulate_kernel, dim3((unsigned)((x_elems / 4 + 256) / 256)), dim3(256), 0, s, dx, tmp,
                           (long)x_elems);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) rc = set_hip_error(e, "accumulate kernel launch");
    }
    const int rc2 = tmp ? workspace_free(tmp, s) : NZHIP_OK;
    return rc ? rc : rc2;
}

namespace nzhip {

// The same tile with 16-byte accesses (HW a multiple of 4, 16-byte aligned tensors): a thread owns four adjacent pixels
// of channels oc and oc + 16, every element still one chain over ascending n (the same sums, bit for bit); two images'
// loads are in flight at a time.
template <bool MASK>
__global__ __launch_bounds__(256) void conv_bias_grad_vec_kernel(float* __restrict__ dbias, const float* __restrict__ dz, int N,
                                                                 int O, long HW, float* __restrict__ dz_out,
                                                                 const float* __restrict__ y) {
    __shared__ float tile[64][33];                               // [pixel][channel]
    const long p0 = (long)blockIdx.x * 64;
    const int o0 = blockIdx.y * 32;
    {
        const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
#pragma unroll
        for (int r = 0; r < 64; r += 8) {
            const long p = p0 + ty + r;
            const int o = o0 + tx;
            tile[ty + r][tx] = (p < HW && o < O) ? dbias[p * O + o] : 0.f;
        }
    }
    __syncthreads();
    const int pq = threadIdx.x & 15, oc = threadIdx.x >> 4;      // pixels 4 pq .. 4 pq + 3, channels oc and oc + 16
    const long p = p0 + 4 * pq;
    float acc[2][4];
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
        for (int e = 0; e < 4; e++) acc[h][e] = tile[4 * pq + e][oc + 16 * h];
    if (p < HW) {                                                // HW % 4 == 0: the four pixels are inside together
        const bool live[2] = {o0 + oc < O, o0 + oc + 16 < O};
        const long plane = HW, image = (long)O * HW;
        const long at0 = (long)(o0 + oc) * plane + p;
        auto step = [&](const int n) {
#pragma unroll
            for (int h = 0; h < 2; h++)
                if (live[h]) {
                    const long at = (long)n * image + at0 + (long)h * 16 * plane;
                    floatx4 g = *reinterpret_cast<const floatx4*>(dz + at);
                    if (MASK) {
                        const floatx4 yy = *reinterpret_cast<const floatx4*>(y + at);
#pragma unroll
                        for (int e = 0; e < 4; e++) g[e] = yy[e] > 0.f ? g[e] : 0.f;
                        *reinterpret_cast<floatx4*>(dz_out + at) = g;
                    }
#pragma unroll
                    for (int e = 0; e < 4; e++) acc[h][e] += g[e];
                }
        };
        int n = 0;
        for (; n + 2 <= N; n += 2) {
            step(n);
            step(n + 1);
        }
        if (n < N) step(n);
    }
    __syncthreads();
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
        for (int e = 0; e < 4; e++) tile[4 * pq + e][oc + 16 * h] = acc[h][e];
    __syncthreads();
    {
        const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
#pragma unroll
        for (int r = 0; r < 64; r += 8) {
            const long pp = p0 + ty + r;
            const int o = o0 + tx;
            if (pp < HW && o < O) dbias[pp * O + o] = tile[ty + r][tx];
        }
    }
}

}  // namespace nzhip

/* Gradient of the reference's Conv2d bias parameter ([1,1,H_out*W_out,O], added to the matmul result before
 * Col2Img): dbias[p][o] += sum over n of dz[n][o][p], dz being the gradient of the convolution output in NCHW.
 * One kernel for Col2ImgNode::backward + AddNode::backward (src/Nodes.cu:660-665, 99-146). */
extern "C" int nzhip_conv2d_backward_bias(float* dbias, const float* dz, size_t N, size_t O, size_t HW, void* stream) {
    if (!dbias || !dz) return set_error(NZHIP_E_INVALID, "nzhip_conv2d_backward_bias: null pointer");
    if (N == 0 || O == 0 || HW == 0) return NZHIP_OK;
    if (N > 0x7fffffff || O > 0x7fffffff || (O + 31) / 32 > 65535 || (HW + 63) / 64 > 0x7fffffffull)
        return set_error(NZHIP_E_UNSUPPORTED, "nzhip_conv2d_backward_bias: extent too large");
    dim3 grid((unsigned)((HW + 63) / 64), (unsigned)((O + 31) / 32));
    const bool vec = HW % 4 == 0 && (reinterpret_cast<uintptr_t>(dz) & 15) == 0;
    hipLaunchKernelGGL(vec ? conv_bias_grad_vec_kernel<false> : conv_bias_grad_kernel<false>, grid, dim3(256), 0,
                       reinterpret_cast<hipStream_t>(stream), dbias, dz, (int)N, (int)O, (long)HW, static_cast<float*>(nullptr),
                       static_cast<const float*>(nullptr));
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? NZHIP_OK : set_hip_error(e, "conv_bias_grad kernel launch");
}

/* The same with the ReLU gradient in front (Conv2d followed by ReLU): dz[n][o][p] = y[n][o][p] > 0 ? dy[n][o][p] : 0
 * is written out (ReLUNode::backward, src/Nodes.cu:357-364) and dbias[p][o] += sum over n of dz[n][o][p] in the same
 * pass, so the masked gradient is not read back for the bias. dz must not overlap y or dy. */
extern "C" int nzhip_conv2d_backward_relu_bias(float* dz, float* dbias, const float* y, const float* dy, size_t N, size_t O,
                                               size_t HW, void* stream) {
    if (!dz || !dbias || !y || !dy) return set_error(NZHIP_E_INVALID, "nzhip_conv2d_backward_relu_bias: null pointer");
    if (N == 0 || O == 0 || HW == 0) return NZHIP_OK;
    if (N > 0x7fffffff || O > 0x7fffffff || (O + 31) / 32 > 65535 || (HW + 63) / 64 > 0x7fffffffull)
        return set_error(NZHIP_E_UNSUPPORTED, "nzhip_conv2d_backward_relu_bias: extent too large");
    dim3 grid((unsigned)((HW + 63) / 64), (unsigned)((O + 31) / 32));
    const bool vec = HW % 4 == 0 && ((reinterpret_cast<uintptr_t>(dz) | reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(dy)) & 15) == 0;
    hipLaunchKernelGGL(vec ? conv_bias_grad_vec_kernel<true> : conv_bias_grad_kernel<true>, grid, dim3(256), 0,
                       reinterpret_cast<hipStream_t>(stream), dbias, dy, (int)N, (int)O, (long)HW, dz, y);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? NZHIP_OK : set_hip_error(e, "conv_bias_grad (masked) kernel launch");
}

// dw[i] += P[0][i] + P[1][i] + ... (ascending, then added to dw once): the per-image products of the 1x1 weight gradient
static __global__ __launch_bounds__(256) void dw_add_members_kernel(float* __restrict__ dw, const float* __restrict__ P, int members, long n) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float sum = 0.f;
    for (int m = 0; m < members; m++) sum += P[(long)m * n + i];
    dw[i] += sum;
}

// Weight gradient of a 1x1, stride 1, unpadded convolution: its column matrix is x itself with pixels and channels
// swapped, so MatMulNode::backward's dB += A^T * dC (src/Nodes.cu:169-182) is, per image,
//   dw[c][o] += sum over pixels of f16(x[n][c][pixel]) * f16(dy[n][o][pixel]),
// a product of two operands that both have the contraction contiguous. Per-sample weights: one batched product that
// reads dw as its bias matrix and writes it back (every element is read and written by the same thread). Shared
// weights: the per-image products go to a workspace and are added in ascending image order.
static int conv1x1_backward_weights(float* dw, const float* x, const float* dy, size_t N, size_t C, size_t HW, size_t O,
                                    bool shared, hipStream_t s) {
    nzhip_gemm_desc g = {};
    g.A = x; g.M = (int64_t)C; g.K = (int64_t)HW; g.lda = (int64_t)HW; g.a_layout = NZHIP_LAYOUT_ROW;
    g.B = dy; g.N = (int64_t)O; g.ldb = (int64_t)HW; g.b_layout = NZHIP_LAYOUT_TRANS;     // dy[n] is [O, pixels]: B^T as stored
    g.ldc = (int64_t)O;
    g.batch_n = (int64_t)N; g.batch_c = 1;
    g.a_stride_n = (int64_t)(C * HW); g.b_stride_n = (int64_t)(O * HW); g.c_stride_n = (int64_t)(C * O);
    g.activation = NZHIP_ACT_NONE;
    if (!shared || N == 1) {
        g.C = dw;
        g.bias = dw; g.bias_stride_n = (int64_t)(C * O); g.bias_stride_row = (int64_t)O; g.bias_stride_col = 1;
        return nzhip_gemm(&g, s);
    }
    float* P = nullptr;
    if (int rc = workspace_alloc(reinterpret_cast<void**>(&P), N * C * O * sizeof(float), s)) return rc;
    g.C = P;
    int rc = nzhip_gemm(&g, s);
    if (rc == NZHIP_OK) {
        const long n = (long)(C * O);
        hipLaunchKernelGGL(dw_add_members_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, dw, P, (int)N, n);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) rc = set_hip_error(e, "dw_add_members kernel launch");
    }
    const int rc2 = workspace_free(P, s);
    return rc ? rc : rc2;
}

namespace nzhip {

// ---- weight gradient for any kernel extent, stride and padding ---------------------------------------------------
// dW[(c, r, s)][o] = sum over pixels of f16(x[c][ho*stride - pad + r][wo*stride - pad + s]) * f16(dy[o][ho][wo]): a product
// whose contraction runs over the output pixels, with the column matrix of the reference's chain (Img2ColNode::forward,
// src/Nodes.cu:605-630, as A of MatMulNode::backward's dB += A^T dC, :169-182) gathered from LDS instead of written to
// memory. A workgroup owns up to 128 (channel, tap) rows (as many whole channels as fit) x 64 output channels and a band
// of output rows of one image; per segment of 128 output pixels (SR rows x SW columns, SW the power of two from 16 to 128
// that covers the output width or 128) it stages the input rows of its channels that the segment touches (zero outside
// the image) and the dy segment in LDS as fp16, then runs eight 32x32x16 MFMA steps per wave. The A fragment of a lane is eight pixels of one (c, r, s) row, `stride`
// elements apart in the staged input row: eight 16-bit LDS reads, which is what makes every tap offset and stride
// one code path. Band sums go to a workspace and are added in ascending order by conv_dwg_reduce_kernel.
constexpr int DWG_PX = 128, DWG_OT = 128, DWG_ROWS = 128, DWG_ZPITCH = DWG_PX + 8, DWG_NB = DWG_OT / 32;

struct ConvDwGenArgs {
    const float* x;        // [N, C, H, W]
    const float* dy;       // [N, O, Ho, Wo]
    float* partial;        // [chunk][o_tile][image][band][DWG_ROWS][DWG_OT]
    int C, H, W, O, Ho, Wo, Kh, Kw, stride, pad;
    int cc;                // channels per workgroup
    int pw;                // staged columns per input row (a multiple of 4 for the vector path)
    int shift;             // staged column 0 is image column wo0 * stride - pad - shift (vector path: 16-byte aligned)
    int sw_log;            // log2 of the segment width SW; a segment is 128 / SW output rows x SW output columns
    int span;              // staged input rows per channel: (128 / SW - 1) * stride + Kh
    int bands, band_rows, n_images;
    int ipw, n_groups;     // images per workgroup and groups of that many images (partial sums: one region per group and band)
    float* dw_direct;      // not null: one workgroup per (image, tile) and per-sample weights -- its sums are the whole
    long dw_stride;        // gradient of that tile, added straight into dW[image] (dw_stride floats apart), no partial sums
};

// Eight waves: a workgroup owns up to 256 rows (channel, tap) x 128 output channels, and the requests for the NEXT
// segment are issued before the current one multiplies. A thread's share of a
// segment is a fixed set of 16-byte pieces (DWG8_XMAX of the input rows, 8 of dy) whose place in the tile does not
// depend on the segment, so the index arithmetic is done once; per segment only the image row and column move.
// Requests are unconditional (clamped addresses, zero selected when the piece is stored), so the compiler's waits
// stay exact; the last step requests its own segment once more instead of branching.
constexpr int DWG8_ROWS = 256, DWG8_XMAX = 7, DWG8_THREADS = 512;

// XP: 16-byte pieces of the staged input rows per thread (the tile has at most 512 XP of them)
// S1: stride 1. A lane's eight pixels are then eight consecutive halfs of a staged row: five dword reads and four
// v_alignbit (by 0 or 16 bits, the parity of the lane's tap column) instead of eight 16-bit reads.
// VEC: rows of x and dy are whole 16-byte pieces (W and Wo multiples of 4, aligned tensors); otherwise a piece's four
// columns are loaded one by one with their own bounds (14-wide images ...).
// A workgroup walks the segments of its band in p.ipw consecutive images (small images: one segment each, and one
// set of partial sums per group of images instead of one per image).
template <int XP, bool S1, bool VEC>
__global__ __launch_bounds__(DWG8_THREADS) void conv_dwg8_kernel(const ConvDwGenArgs p) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    _Float16* xs = reinterpret_cast<_Float16*>(lds);                                   // [cc * span][pw]
    _Float16* zs = xs + ((p.cc * p.span * p.pw + 7) & ~7);                              // [DWG_OT][DWG_ZPITCH]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lh = lane >> 5;
    const int band = blockIdx.x % p.bands, group = blockIdx.x / p.bands;
    const int img0 = group * p.ipw, n_img = (p.n_images - img0) < p.ipw ? (p.n_images - img0) : p.ipw;
    const int c0 = blockIdx.y * p.cc, o0 = blockIdx.z * DWG_OT;
    const int taps = p.Kh * p.Kw;
    const int nch = (p.C - c0) < p.cc ? (p.C - c0) : p.cc;
    const int h_begin = band * p.band_rows;
    const int h_end = (h_begin + p.band_rows) < p.Ho ? (h_begin + p.band_rows) : p.Ho;
    const long x_image = (long)p.C * p.H * p.W, z_image = (long)p.O * p.Ho * p.Wo;
    const float* ximg0 = p.x + (long)c0 * p.H * p.W;
    const float* zimg0 = p.dy + (long)o0 * p.Ho * p.Wo;

    floatx16 acc[DWG_NB];
#pragma unroll
    for (int j = 0; j < DWG_NB; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[j][r] = 0.f;

    const int m = wave * 32 + li;
    const bool row_live = m < nch * taps;
    const int mc = row_live ? m / taps : 0, mt = row_live ? m % taps : 0;
    const int a_base = (mc * p.span + mt / p.Kw) * p.pw + mt % p.Kw + p.shift + 8 * lh * p.stride;
    const bool wave_live = wave * 32 < nch * taps;                                     // wave-uniform
    const int SW = 1 << p.sw_log, SR = DWG_PX >> p.sw_log;
    const int segs = (p.Wo + SW - 1) >> p.sw_log;

    // this thread's pieces of the staged input rows: piece e = tid + 512 k is 4 columns of staged row e / pw4
    const int pw4 = p.pw >> 2, n4 = nch * p.span * pw4;
    int xoff[XP], xrq[XP];
#pragma unroll
    for (int k = 0; k < XP; k++) {
        const int e = tid + DWG8_THREADS * k;
        const int row = e / pw4, q = e - row * pw4;
        const int c = row / p.span, r = row - c * p.span;
        xoff[k] = (c * p.H + r) * p.W + 4 * q;
        xrq[k] = e < n4 ? (r | (q << 16)) : -1;
    }
    // ... and of the dy segment: output channel tid / 32 + 16 k, pixels 4 (tid % 32) .. + 3 of the segment
    const int zo = tid >> 5, zk = (tid & 31) * 4;
    const int zkr = zk >> p.sw_log, zkc = zk & (SW - 1);

    const int xn = (n4 + DWG8_THREADS - 1) / DWG8_THREADS;                             // pieces per thread that exist at all (uniform)
    floatx4 xr[XP], zr[8];
    constexpr int MB = VEC ? 1 : 4;                       // mask bits per piece: which of its columns lie inside the images
    unsigned xin = 0, zin = 0;
    const float* ximg = ximg0 + (long)img0 * x_image;     // the image being requested
    const float* zimg = zimg0 + (long)img0 * z_image;
    auto request = [&](int ho, int wo0) {
        const int hb = ho * p.stride - p.pad, wf = wo0 * p.stride - p.pad - p.shift;
        const int corner = hb * p.W + wf;
        xin = 0; zin = 0;
#pragma unroll
        for (int k = 0; k < XP; k++) {
            if (k < xn) {
                const int h = hb + (xrq[k] & 0xffff), w = wf + 4 * (xrq[k] >> 16);
                const bool row_in = xrq[k] >= 0 && h >= 0 && h < p.H;
                if (VEC) {
                    const bool in = row_in && w >= 0 && w < p.W;
                    xr[k] = *reinterpret_cast<const floatx4*>(ximg + (in ? xoff[k] + corner : 0));
                    xin |= (in ? 1u : 0u) << k;
                } else {
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const bool in = row_in && w + j >= 0 && w + j < p.W;
                        xr[k][j] = ximg[in ? xoff[k] + corner + j : 0];
                        xin |= (in ? 1u : 0u) << (MB * k + j);
                    }
                }
            }
        }
        const bool zrow = ho + zkr < h_end;
        const long zpos = (long)(zrow ? ho + zkr : 0) * p.Wo + wo0 + zkc;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const int o = zo + 16 * k;
            const bool o_in = zrow && o0 + o < p.O;
            if (VEC) {
                const bool in = o_in && wo0 + zkc < p.Wo;
                zr[k] = *reinterpret_cast<const floatx4*>(zimg + (in ? (long)o * p.Ho * p.Wo + zpos : 0));
                zin |= (in ? 1u : 0u) << k;
            } else {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const bool in = o_in && wo0 + zkc + j < p.Wo;
                    zr[k][j] = zimg[in ? (long)o * p.Ho * p.Wo + zpos + j : 0];
                    zin |= (in ? 1u : 0u) << (MB * k + j);
                }
            }
        }
    };
    auto deposit = [&]() {
#pragma unroll
        for (int k = 0; k < XP; k++) {
            if (k < xn) {
                half4_t hv;
#pragma unroll
                for (int j = 0; j < 4; j++) hv[j] = (xin >> (MB * k + (VEC ? 0 : j)) & 1) ? (_Float16)xr[k][j] : (_Float16)0.f;   // VEC: all four or none
                if (xrq[k] >= 0) *reinterpret_cast<half4_t*>(xs + 4 * (tid + DWG8_THREADS * k)) = hv;
            }
        }
#pragma unroll
        for (int k = 0; k < 8; k++) {
            half4_t hv;
#pragma unroll
            for (int j = 0; j < 4; j++) hv[j] = (zin >> (MB * k + (VEC ? 0 : j)) & 1) ? (_Float16)zr[k][j] : (_Float16)0.f;
            *reinterpret_cast<half4_t*>(zs + (zo + 16 * k) * DWG_ZPITCH + zk) = hv;
        }
    };

    const int n_steps = n_img > 0 ? n_img * ((h_end - h_begin + SR - 1) / SR * segs) : 0;
    int ho = h_begin, seg = 0;
    if (n_steps > 0) request(ho, 0);
    for (int step = 0; step < n_steps; step++) {
        deposit();
        __syncthreads();
        {   // the next segment (the last step asks for its own again: no branch around the requests)
            int nseg = seg + 1, nho = ho;
            bool next_image = false;
            if (nseg == segs) { nseg = 0; nho += SR; }
            if (nho >= h_end) { nho = h_begin; next_image = true; }
            if (step + 1 == n_steps) { nseg = seg; nho = ho; next_image = false; }
            if (next_image) { ximg += x_image; zimg += z_image; }
            request(nho, nseg * SW);
            seg = nseg; ho = nho;
        }
        if (wave_live) {
            // two fragment sets: the reads of k step ks + 1 are issued before the MFMAs of step ks
            half8_t af[2], bf[2][DWG_NB];
            auto fragments = [&](int ks, int set) {
                if (S1) {
                    // (segment row) * pw and the column of the k step are even, so the parity is a_base's
                    const int eo = a_base + ((ks * 16) >> p.sw_log) * p.pw + ((ks * 16) & (SW - 1));
                    const unsigned* dp = reinterpret_cast<const unsigned*>(xs) + (eo >> 1);
                    const unsigned sh = (a_base & 1) * 16;
                    unsigned d[5];
#pragma unroll
                    for (int j = 0; j < 5; j++) d[j] = dp[j];
                    union { unsigned u[4]; half8_t h; } pack;
#pragma unroll
                    for (int j = 0; j < 4; j++) pack.u[j] = __builtin_amdgcn_alignbit(d[j + 1], d[j], sh);
                    af[set] = pack.h;
                } else {
                    const _Float16* ap = xs + a_base + (((ks * 16) >> p.sw_log) * p.pw + ((ks * 16) & (SW - 1))) * p.stride;
#pragma unroll
                    for (int j = 0; j < 8; j++) af[set][j] = ap[j * p.stride];
                }
#pragma unroll
                for (int j = 0; j < DWG_NB; j++)
                    bf[set][j] = *reinterpret_cast<const half8_t*>(zs + (j * 32 + li) * DWG_ZPITCH + ks * 16 + lh * 8);
            };
            if (VEC) {
                fragments(0, 0);
#pragma unroll
                for (int ks = 0; ks < DWG_PX / 16; ks++) {
                    if (ks + 1 < DWG_PX / 16) fragments(ks + 1, (ks + 1) & 1);
#pragma unroll
                    for (int j = 0; j < DWG_NB; j++)
                        acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[ks & 1], bf[ks & 1][j], acc[j], 0, 0, 0);
                }
            } else {
                // the per-column loads of this variant hold four address registers per piece: one fragment set
#pragma unroll 2
                for (int ks = 0; ks < DWG_PX / 16; ks++) {
                    fragments(ks, 0);
#pragma unroll
                    for (int j = 0; j < DWG_NB; j++)
                        acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[0], bf[0][j], acc[j], 0, 0, 0);
                }
            }
        }
        __syncthreads();
    }
    // accumulator (block j, register r): row 32 wave + (r >> 2) * 8 + lh * 4 + (r & 3), column 32 j + li
    if (p.dw_direct) {
        float* dst = p.dw_direct + (long)group * p.dw_stride + (long)c0 * taps * p.O + o0;
        if (wave_live) {
            // all of a column block's old values requested before the first is added and stored (a store might alias
            // a later load as far as the compiler knows, which would put one memory round trip behind the other)
#pragma unroll
            for (int j = 0; j < DWG_NB; j++) {
                const int col = j * 32 + li;
                float old[16];
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int row = wave * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
                    const bool ok = row < nch * taps && o0 + col < p.O;
                    old[r] = ok ? dst[(long)row * p.O + col] : 0.f;
                }
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int row = wave * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
                    if (row < nch * taps && o0 + col < p.O) dst[(long)row * p.O + col] = old[r] + acc[j][r];
                }
            }
        }
        return;
    }
    float* out = p.partial + ((((long)blockIdx.y * gridDim.z + blockIdx.z) * p.n_groups + group) * p.bands + band) * (DWG8_ROWS * DWG_OT);
    if (wave_live) {
#pragma unroll
        for (int j = 0; j < DWG_NB; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int row = wave * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
                out[row * DWG_OT + j * 32 + li] = acc[j][r];
            }
    }
}

// dW[b][(c0 + c) * taps + t][o0 + o] += the S partial regions of weight copy b, in ascending order (per-sample weights:
// the bands of image b; shared weights: images x bands).
__global__ __launch_bounds__(256) void conv_dwg_reduce_kernel(float* __restrict__ dW, const float* __restrict__ P, int S, int C, int O,
                                                              int taps, int cc, int n_otiles, long group_stride_P, long group_stride_dW,
                                                              int region_rows) {
    const int chunk = blockIdx.y / n_otiles, ot = blockIdx.y % n_otiles, b = blockIdx.z;
    const int c0 = chunk * cc, o0 = ot * DWG_OT;
    const int nch = (C - c0) < cc ? (C - c0) : cc;
    const int t = blockIdx.x * 256 + threadIdx.x;
    const int row = t / DWG_OT, col = t % DWG_OT;
    if (row >= nch * taps || o0 + col >= O) return;
    const float* src = P + (long)blockIdx.y * gridDim.z * group_stride_P + (long)b * group_stride_P + t;
    float sum = 0.f;
    for (int s = 0; s < S; s++) sum += src[(long)s * region_rows * DWG_OT];
    dW[(long)b * group_stride_dW + ((long)c0 * taps + row) * O + o0 + col] += sum;
}

// Row bands per image for the weight-gradient kernels: with `units` (chunk, output tile, image) triples and `resident`
// workgroups running at a time, the number of bands that minimises rounds x (segments of a band + the cost of a
// workgroup's result stores, in segment times). More bands even the rounds out, fewer keep the partial sums small.
// `region_cost`: what one more set of partial sums costs the reduction that follows, in segment times (0 leaves it out).
static int dwg_pick_bands(long units, long resident, long row_steps, long segs, double store_cost, double region_cost = 0.0,
                          double* cost_out = nullptr) {
    int best = 1;
    double best_cost = 1e300;
    const long max_bands = row_steps < 64 ? row_steps : 64;
    for (long b = 1; b <= max_bands; b++) {
        const long steps = (row_steps + b - 1) / b;                   // row steps of the largest band
        const long bands = (row_steps + steps - 1) / steps;
        if (bands != b) continue;                                     // the same split as a smaller count
        const long rounds = (units * bands + resident - 1) / resident;
        const double cost = (double)rounds * ((double)steps * (double)segs + store_cost) + (double)(units * bands) * region_cost;
        if (cost < best_cost - 1e-9) { best_cost = cost; best = (int)b; }
    }
    if (cost_out) *cost_out = best_cost;
    return best;
}

// Ho, Wo: the extents of dy as it lies in memory. Wo may exceed what (W, K_w, stride, pad) give when dy is a copy with
// zero-filled columns appended (below): those columns add nothing to any sum.
static int conv_dw_generic_run(float* dw, const float* x, const float* dy, size_t N, size_t C, size_t H, size_t W, size_t O,
                               size_t K_h, size_t K_w, size_t stride, size_t pad, size_t Ho, size_t Wo, bool shared, hipStream_t s) {
    const size_t taps = K_h * K_w;
    const bool vec = W % 4 == 0 && Wo % 4 == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(dy)) & 15) == 0;
    int cc = (int)(DWG8_ROWS / taps);
    if (cc > (int)C) cc = (int)C;
    // 16-byte pieces: the staged window starts at a multiple of four columns, `shift` columns left of the first one needed
    // (128 * stride is a multiple of 4, so the shift is the same for every segment)
    const int shift = vec ? (int)(((4 - (long)(pad % 4)) % 4 + 4) % 4) : 0;
    int sw_log = 7;                                                   // segment width: 16 .. 128, covering the output width
    while (sw_log > 4 && (size_t)(1 << (sw_log - 1)) >= Wo) sw_log--;
    const int SW = 1 << sw_log, SR = DWG_PX / SW;
    const int span = (int)((SR - 1) * stride + K_h);
    int pw = (int)((SW - 1) * stride + K_w) + shift;
    pw = (pw + 3) / 4 * 4;
    // staged input rows + dy segment: at most 96 KiB, and DWG8_XMAX 16-byte pieces of input rows per thread
    auto too_big = [&](int c) {
        if (((size_t)c * span * pw + 8) * 2 + (size_t)DWG_OT * DWG_ZPITCH * 2 > 96 * 1024) return true;
        return (size_t)c * span * (pw / 4) > (size_t)DWG8_THREADS * DWG8_XMAX;
    };
    while (cc > 1 && too_big(cc)) cc--;
    if (too_big(cc)) return NZHIP_E_UNSUPPORTED;
    if ((size_t)cc * H * W + (size_t)(stride * DWG_PX + K_h) * W >= 0x7fffffffull) return NZHIP_E_UNSUPPORTED;   // int offsets in the kernel
    const size_t lds_bytes = (((size_t)cc * span * pw + 7) & ~(size_t)7) * 2 + (size_t)DWG_OT * DWG_ZPITCH * 2;
    const int chunks = (int)((C + cc - 1) / cc), otiles = (int)((O + DWG_OT - 1) / DWG_OT);
    if (chunks > 65535 || otiles > 65535) return NZHIP_E_UNSUPPORTED;
    // A workgroup takes a band of segment rows of one image, or -- small images, shared weights -- all segments of several
    // images: whichever split minimises rounds x (segments per workgroup + the cost of its result stores).
    const long row_steps = ((long)Ho + SR - 1) / SR, segs = ((long)Wo + SW - 1) / SW;
    const long resident = (long)device_cu_count();
    const long tiles = (long)chunks * otiles;
    // A set of partial sums (256 rows x 128 channels of fp32, 128 KiB) is read back by the reduction at about 0.03 us,
    // a hundredth of the 2.5-3 us a segment takes: that decides between splits of nearly equal rounds (16 x 256 x 56 x 56 -> 256: 4 bands of 7 row steps left
    // 1280 sets, 168 MB, and 46 us of reduction behind a 154 us kernel).
    const double region_cost = 0.011;
    double best = 0.0;
    int bands = dwg_pick_bands(tiles * (long)N, resident, row_steps, segs, 3.0, region_cost, &best), ipw = 1;
    if (!shared && bands > 1) {
        // one band per image needs no partial sums and no reduction at all (below): its cost without those
        const long units = tiles * (long)N;
        const double one = (double)((units + resident - 1) / resident) * ((double)row_steps * (double)segs + 3.0) - 1.7;
        if (one <= best) bands = 1;
    }
    if (shared && N > 1) {
        for (long g = 2; g <= (long)N && g <= 64; g++) {
            const long groups = ((long)N + g - 1) / g;
            if ((groups - 1) * g >= (long)N) continue;
            const double cost = (double)((tiles * groups + resident - 1) / resident) * ((double)g * (double)row_steps * (double)segs + 3.0) +
                                (double)(tiles * groups) * region_cost;
            if (cost < best - 1e-9) { best = cost; ipw = (int)g; bands = 1; }
        }
    }
    const int band_rows = (int)((row_steps + bands - 1) / bands) * SR;
    bands = (int)((Ho + band_rows - 1) / band_rows);
    const int n_groups = (int)((N + ipw - 1) / ipw);
    if ((size_t)n_groups * (size_t)bands > 0x7fffffffull) return NZHIP_E_UNSUPPORTED;
    const size_t regions = (size_t)chunks * otiles * n_groups * bands;
    // Per-sample weights and one workgroup per (image, tile): its sums are that tile's whole gradient and go straight
    // into dW[image] -- no partial sums written and read back (16 x 512 x 7 x 7 -> 512 with a weight copy per image: 302 MB
    // of dW traffic instead of 604 MB).
    const bool direct = !shared && bands == 1 && ipw == 1;
    float* partial = nullptr;
    if (!direct)
        if (int rc = workspace_alloc(reinterpret_cast<void**>(&partial), regions * DWG8_ROWS * DWG_OT * sizeof(float), s)) return rc;
    ConvDwGenArgs a;
    a.x = x; a.dy = dy; a.partial = partial;
    a.dw_direct = direct ? dw : nullptr; a.dw_stride = (long)(C * taps * O);
    a.C = (int)C; a.H = (int)H; a.W = (int)W; a.O = (int)O; a.Ho = (int)Ho; a.Wo = (int)Wo;
    a.Kh = (int)K_h; a.Kw = (int)K_w; a.stride = (int)stride; a.pad = (int)pad;
    a.cc = cc; a.pw = pw; a.shift = shift; a.sw_log = sw_log; a.span = span; a.bands = bands; a.band_rows = band_rows; a.n_images = (int)N;
    a.ipw = ipw; a.n_groups = n_groups;
    const size_t x_pieces = ((size_t)cc * span * (pw / 4) + DWG8_THREADS - 1) / DWG8_THREADS;
    auto pick = [&](auto vec_tag) {
        constexpr bool V = decltype(vec_tag)::value;
        return stride == 1 ? (x_pieces <= 4 ? conv_dwg8_kernel<4, true, V> : conv_dwg8_kernel<DWG8_XMAX, true, V>)
                           : (x_pieces <= 4 ? conv_dwg8_kernel<4, false, V> : conv_dwg8_kernel<DWG8_XMAX, false, V>);
    };
    auto kfn = vec ? pick(std::true_type{}) : pick(std::false_type{});
    int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kfn), (int)lds_bytes, "hipFuncSetAttribute(conv_dwg)");
    if (rc == NZHIP_OK) {
        hipLaunchKernelGGL(kfn, dim3((unsigned)(n_groups * bands), (unsigned)chunks, (unsigned)otiles), dim3(DWG8_THREADS), lds_bytes, s, a);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) rc = set_hip_error(e, "conv_dwg kernel launch");
    }
    if (rc == NZHIP_OK && !direct) {
        const int S = shared ? n_groups * bands : bands, groups = shared ? 1 : (int)N;
        const long per_group = (long)S * DWG8_ROWS * DWG_OT;
        // partial regions of one (chunk, o_tile) are contiguous: [image group][band]; a weight copy's regions start at b * S
        dim3 grid((unsigned)((DWG8_ROWS * DWG_OT + 255) / 256), (unsigned)(chunks * otiles), (unsigned)groups);
        hipLaunchKernelGGL(conv_dwg_reduce_kernel, grid, dim3(256), 0, s, dw, partial, S, (int)C, (int)O, (int)taps, cc, otiles,
                           per_group, (long)(C * taps * O), DWG8_ROWS);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) rc = set_hip_error(e, "conv_dwg_reduce kernel launch");
    }
    const int rc2 = partial ? workspace_free(partial, s) : NZHIP_OK;
    return rc ? rc : rc2;
}

// Rows of x or dy that are not whole 16-byte pieces (14-wide images, 28-wide ones at stride 2) put the kernel on four
// loads and four bounds per piece and one fragment set. From about 3 GFLOP on, zero-filled copies with rows of the next
// multiple of 4 pay for themselves; appended zeros of dy add nothing, and the columns appended to x are the zeros its
// bounds check would have produced (16 x 512 x 14 x 14 -> 512: 89 -> 56 us + two copies of 6 MB; 16 x 192 x 35 x 35 -> 192:
// 123 -> 66; 16 x 256 x 28 x 28 -> 256 at stride 2: 55 -> 33). NZHIP_CONV_WIDEN (read per call): 0 never, 1 always.
static int conv_dw_generic(float* dw, const float* x, const float* dy, size_t N, size_t C, size_t H, size_t W, size_t O,
                           size_t K_h, size_t K_w, size_t stride, size_t pad, bool shared, hipStream_t s) {
    const size_t Ho = (H + 2 * pad - K_h) / stride + 1, Wo = (W + 2 * pad - K_w) / stride + 1;
    const char* widen_env = getenv("NZHIP_CONV_WIDEN");
    const double flops = 2.0 * (double)N * (double)Ho * (double)Wo * (double)C * (double)(K_h * K_w) * (double)O;
    const size_t Ww = (W + 3) / 4 * 4, Wow = (Wo + 3) / 4 * 4;
    const bool widen = (W % 4 != 0 || Wo % 4 != 0) && (widen_env ? atoi(widen_env) != 0 : flops >= 3e9) && H * Ww < 0x3fffffffull &&
                       N * C * H < 0x7fffffffull && N * O * Ho < 0x7fffffffull;
    if (!widen) return conv_dw_generic_run(dw, x, dy, N, C, H, W, O, K_h, K_w, stride, pad, Ho, Wo, shared, s);
    float* x_wide = nullptr;
    float* dy_wide = nullptr;
    int rc = NZHIP_OK;
    if (W % 4 != 0) rc = widen_rows(&x_wide, x, N * C * H, W, s);
    if (rc == NZHIP_OK && Wo % 4 != 0) rc = widen_rows(&dy_wide, dy, N * O * Ho, Wo, s);
    if (rc == NZHIP_OK)
        rc = conv_dw_generic_run(dw, x_wide ? x_wide : x, dy_wide ? dy_wide : dy, N, C, H, x_wide ? Ww : W, O, K_h, K_w, stride, pad, Ho,
                                 dy_wide ? Wow : Wo, shared, s);
    const int rc2 = dy_wide ? workspace_free(dy_wide, s) : NZHIP_OK;
    const int rc3 = x_wide ? workspace_free(x_wide, s) : NZHIP_OK;
    return rc ? rc : (rc2 ? rc2 : rc3);
}

}  // namespace nzhip

/* Gradient of nzhip_conv2d_forward with respect to the weights, without the column matrix the reference's
 * chain needs (Img2ColNode::forward output as A in MatMulNode::backward, dB += A^T * dC, src/Nodes.cu:169-182):
 *   dW[wb][(c, r, s)][o] += sum over h, w (and over n when the weights are shared) of
 *                           f16(x[n][c][h+r-pad][w+s-pad]) * f16(dy[n][o][h][w]) */
extern "C" int nzhip_conv2d_backward_weights(float* dw, const float* x, const float* dy, size_t N, size_t C, size_t H,
                                             size_t W, size_t O, size_t K_h, size_t K_w, size_t stride, size_t pad,
                                             size_t w_batch, void* stream) {
    if (!dw || !x || !dy) return set_error(NZHIP_E_INVALID, "nzhip_conv2d_backward_weights: null pointer");
    if (w_batch != 1 && w_batch != N) return set_error(NZHIP_E_SHAPE, "Shapes are not broadcast compatible.");
    // Images of fewer than 64 output pixels (7 x 7 outputs of a network's last stage) with shared weights: a product per
    // image has a contraction of 49, and a 128-pixel segment of the gather kernel is mostly padding. The column matrices
    // of all images follow each other in memory as ONE [N pixels, C K_h K_w] matrix, so the reference's own chain
    // (Img2ColNode::forward, then dB += A^T dC of MatMulNode::backward, src/Nodes.cu:605-630, 169-182) becomes one product
    // with the contraction over all pixels of all images: dw += col^T x dy^T (16 x 512 x 14 x 14 -> 512 at stride 2:
    // 91 -> 55 us; 16 x 1024 x 14 x 14 -> 2048 1x1 stride 2: 105 -> 56; 16 x 2048 x 7 x 7 -> 512 1x1: 57 -> 40).
    static const char* dwf_env = getenv("NZHIP_CONV_DW_FOLD");          // benchmarking only: 0 never, 1 wherever it applies
    if (stride != 0 && K_h != 0 && K_w != 0 && H + 2 * pad >= K_h && W + 2 * pad >= K_w && w_batch == 1 && N != 0 && C != 0 && O != 0) {
        const size_t Ho = (H + 2 * pad - K_h) / stride + 1, Wo = (W + 2 * pad - K_w) / stride + 1, P = Ho * Wo, CKK = C * K_h * K_w;
        const bool fits = N * P < 0x3fffffff && CKK < 0x3fffffff && O < 0x3fffffff && N <= 65535 && N * P * CKK <= ((size_t)1 << 27);
        const bool wanted = dwf_env ? atoi(dwf_env) != 0 : (P < 64 && N * P >= 256 && CKK >= 256 && O >= 64 && CKK * O >= 65536);
        if (fits && wanted) {
            hipStream_t s = reinterpret_cast<hipStream_t>(stream);
            float* col = nullptr;
            float* dyt = nullptr;
            if (int rc = workspace_alloc(reinterpret_cast<void**>(&col), N * P * CKK * sizeof(float), s)) return rc;
            if (int rc = workspace_alloc(reinterpret_cast<void**>(&dyt), N * P * O * sizeof(float), s)) {
                workspace_free(col, s);
                return rc;
            }
            int rc = nzhip_im2col(col, x, Ho, Wo, C, K_h, K_w, stride, pad, H, W, N, stream);
            if (rc == NZHIP_OK) rc = nzhip_col2im_backward(dyt, dy, Ho, Wo, O, N, stream);          // [N][pixels][O]
            if (rc == NZHIP_OK) {
                nzhip_gemm_desc g = {};
                g.A = col; g.M = (int64_t)CKK; g.K = (int64_t)(N * P); g.lda = (int64_t)CKK; g.a_layout = NZHIP_LAYOUT_TRANS;   // col holds K x M
                g.B = dyt; g.N = (int64_t)O; g.ldb = (int64_t)O; g.b_layout = NZHIP_LAYOUT_ROW;
                g.C = dw; g.ldc = (int64_t)O;
                g.bias = dw; g.bias_stride_row = (int64_t)O; g.bias_stride_col = 1;                    // dw += ...
                g.batch_n = 1; g.batch_c = 1;
                g.activation = NZHIP_ACT_NONE;
                rc = nzhip_gemm(&g, s);
            }
            const int rc2 = workspace_free(dyt, s), rc3 = workspace_free(col, s);
            return rc ? rc : (rc2 ? rc2 : rc3);
        }
    }
    if (K_h == 1 && K_w == 1 && stride == 1 && pad == 0 && H > 0 && W > 0 && H * W < 0x3fffffff && C < 0x3fffffff &&
        O < 0x3fffffff && N <= 65535 && N * C * O < 0x7fffffffull) {
        if (N == 0 || C == 0 || O == 0) return NZHIP_OK;
        hipStream_t s = reinterpret_cast<hipStream_t>(stream);
        if (conv1x1_wants_wide_planes(H * W, 2.0 * (double)N * (double)(H * W) * (double)C * (double)O,
                                      2.0 * (double)C * (double)O / (double)(C + O))) {   // zero-filled planes of whole 16-byte pieces: the zeros add nothing
            float* x_wide = nullptr;
            float* dy_wide = nullptr;
            int rc = widen_rows(&x_wide, x, N * C, H * W, s);
            if (rc == NZHIP_OK) rc = widen_rows(&dy_wide, dy, N * O, H * W, s);
            if (rc == NZHIP_OK) rc = conv1x1_backward_weights(dw, x_wide, dy_wide, N, C, (H * W + 3) / 4 * 4, O, w_batch == 1, s);
            const int rc2 = dy_wide ? workspace_free(dy_wide, s) : NZHIP_OK;
            const int rc3 = x_wide ? workspace_free(x_wide, s) : NZHIP_OK;
            return rc ? rc : (rc2 ? rc2 : rc3);
        }
        return conv1x1_backward_weights(dw, x, dy, N, C, H * W, O, w_batch == 1, s);
    }
    if (stride == 0 || K_h == 0 || K_w == 0) return set_error(NZHIP_E_INVALID, "nzhip_conv2d_backward_weights: zero stride or kernel extent");
    if (H + 2 * pad < K_h || W + 2 * pad < K_w)
        return set_error(NZHIP_E_SHAPE, "nzhip_conv2d_backward_weights: kernel larger than the padded input");
    if (conv1x1_strided(K_h, K_w, stride, pad, N, C, H, W)) {
        // 1x1 with a stride: the pixels the convolution looked at, gathered once, then the 1x1 stride-1 product
        // (16 x 1024 x 14 x 14 -> 2048 at stride 2: 351 -> 35 us)
        if (N == 0 || C == 0 || O == 0) return NZHIP_OK;
        hipStream_t s = reinterpret_cast<hipStream_t>(stream);
        const size_t Ho = (H - 1) / stride + 1, Wo = (W - 1) / stride + 1;
        float* sub = nullptr;
        if (int rc = conv_subsample(&sub, x, N * C, H, W, Ho, Wo, stride, s)) return rc;
        const int rc = nzhip_conv2d_backward_weights(dw, sub, dy, N, C, Ho, Wo, O, 1, 1, 1, 0, w_batch, stream);
        const int rc2 = workspace_free(sub, s);
        return rc ? rc : rc2;
    }
    // 3x3, stride 1, pad 1 has a kernel of its own, built around 16-byte pieces of rows that are multiples of 8 wide; narrower
    // or odd rows (28-, 14-wide images) are better off on the gather kernel (16 x 256 x 28 x 28 -> 256: 163 us there), and so
    // are images up to 64 wide with 128 or more input channels (16 x 512 x 32 x 32 -> 512: 450 against 150 us; 16 x 128 x
    // 56 x 56 -> 256: 110 against 86), whose 32-channel workgroups re-read the output gradient once per 32 input channels
    static const char* dw_env = getenv("NZHIP_CONV_DW");             // benchmarking only: "gather" / "own" force either where both apply
    const bool prefer_gather = dw_env ? dw_env[0] == 'g' : (W <= 64 && C >= 128);
    const bool own3x3 = K_h == 3 && K_w == 3 && stride == 1 && pad == 1 &&
                        ((W % 8 == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(dy)) & 15) == 0 && !prefer_gather) ||
                         (C <= 4 && O <= 2));
    if (!own3x3) {
        // any other geometry: the gather kernel (up to 128 taps, stride up to 4, extents that fit its index arithmetic)
        const bool fits = K_h * K_w <= (size_t)DWG_ROWS && stride <= 4 && pad < 0x10000 && H < 0x3fffffff && W < 0x3fffffff &&
                          C < 0x3fffffff && O < 0x3fffffff && N <= 65535 && H * W < 0x3fffffffull;
        if (N == 0 || C == 0 || O == 0) return NZHIP_OK;
        const int rc = fits ? conv_dw_generic(dw, x, dy, N, C, H, W, O, K_h, K_w, stride, pad, w_batch == 1,
                                              reinterpret_cast<hipStream_t>(stream))
                            : NZHIP_E_UNSUPPORTED;
        if (rc == NZHIP_E_UNSUPPORTED)
            return set_error(NZHIP_E_UNSUPPORTED,
                             "nzhip_conv2d_backward_weights: more than 128 taps, a stride above 4 or extents beyond the fused kernels (use the column-matrix chain)");
        return rc;
    }
    if (H == 0 || W == 0 || H > 0x3fffffff || W > 0x3fffffff || C > 0x3fffffff || O > 0x3fffffff || N > 65535)
        return set_error(NZHIP_E_UNSUPPORTED, "nzhip_conv2d_backward_weights: extents beyond the fused kernels (use the column-matrix chain)");
    const bool vec = W % 8 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(dy) & 15) == 0;
    if (N == 0 || C == 0 || O == 0) return NZHIP_OK;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (C <= 4 && O <= 2 && W % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(dy) & 15) == 0) {
        // a handful of channels: stream x and dy once, C*9*O running sums per lane
        dim3 grid((unsigned)((W + 255) / 256), (unsigned)((H + 4 * ST_ROWS - 1) / (4 * ST_ROWS)), (unsigned)N);
        const size_t Q = C * 9 * O, per_image = (size_t)grid.x * grid.y * 4;
        if (per_image * N > 0x7fffffffull) return set_error(NZHIP_E_UNSUPPORTED, "nzhip_conv2d_backward_weights: too many strips");
        float* partial = nullptr;
        if (int rc = workspace_alloc(reinterpret_cast<void**>(&partial), per_image * N * Q * sizeof(float), s)) return rc;
#define NZHIP_DWS(OT, CT)                                                                                            \
    hipLaunchKernelGGL((conv3x3_dw_stream_kernel<OT, CT>), grid, dim3(256), 0, s, partial, x, dy, (int)H, (int)W)
        switch ((int)(O * 10 + C)) {
            case 11: NZHIP_DWS(1, 1); break;
            case 12: NZHIP_DWS(1, 2); break;
            case 13: NZHIP_DWS(1, 3); break;
            case 14: NZHIP_DWS(1, 4); break;
            case 21: NZHIP_DWS(2, 1); break;
            case 22: NZHIP_DWS(2, 2); break;
            case 23: NZHIP_DWS(2, 3); break;
            default: NZHIP_DWS(2, 4); break;
        }
#undef NZHIP_DWS
        hipError_t e = hipGetLastError();
        int rc = e == hipSuccess ? NZHIP_OK : set_hip_error(e, "conv3x3_dw_stream kernel launch");
        if (rc == NZHIP_OK) {
            const bool shared = w_batch == 1;
            const int S = (int)(shared ? per_image * N : per_image), groups = shared ? 1 : (int)N;
            hipLaunchKernelGGL(small_dw_reduce_kernel, dim3((unsigned)((Q + 31) / 32), (unsigned)groups), dim3(256), 0, s, dw,
                               partial, S, (int)Q);
            e = hipGetLastError();
            if (e != hipSuccess) rc = set_hip_error(e, "small_dw_reduce kernel launch");
        }
        const int rc2 = workspace_free(partial, s);
        return rc ? rc : rc2;
    }
    const int chunks = (int)((C + DW_CC - 1) / DW_CC), otiles = (int)((O + DW_OT - 1) / DW_OT);
    if (chunks > 65535 || otiles > 65535) return set_error(NZHIP_E_UNSUPPORTED, "nzhip_conv2d_backward_weights: too many channels");
    // one workgroup per CU in total (its LDS footprint leaves room for no second one); a band is a whole
    // number of rows of one image
    const int cus = device_cu_count();
    long want = ((long)cus + (long)chunks * otiles * (long)N - 1) / ((long)chunks * otiles * (long)N);
    if (want < 1) want = 1;
    if (want > (long)H) want = (long)H;
    const int band_rows = (int)((H + want - 1) / want);
    const int bands = (int)((H + band_rows - 1) / band_rows);
    const size_t region = (size_t)DW_CC * 9 * DW_OT;
    const size_t regions = (size_t)chunks * otiles * N * bands;
    if (N * (size_t)bands > 0x7fffffffull) return set_error(NZHIP_E_UNSUPPORTED, "nzhip_conv2d_backward_weights: too many row bands");
    float* partial = nullptr;
    if (int rc = workspace_alloc(reinterpret_cast<void**>(&partial), regions * region * sizeof(float), s)) return rc;
    ConvDwArgs a;
    a.x = x; a.dy = dy; a.partial = partial;
    a.C = (int)C; a.H = (int)H; a.W = (int)W; a.O = (int)O;
    a.bands = bands; a.band_rows = band_rows; a.n_images = (int)N;
    const int lds_bytes = DW_XS_BYTES + DW_ZS_BYTES;
    auto kfn = vec ? conv_dw_kernel<true> : conv_dw_kernel<false>;
    int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kfn), lds_bytes, "hipFuncSetAttribute(conv_dw)");
    if (rc == NZHIP_OK) {
        dim3 grid((unsigned)(N * bands), (unsigned)chunks, (unsigned)otiles);
        hipLaunchKernelGGL(kfn, grid, dim3(256), lds_bytes, s, a);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) rc = set_hip_error(e, "conv_dw kernel launch");
    }
    if (rc == NZHIP_OK) {
        const bool shared = w_batch == 1;
        const int S = shared ? (int)(N * bands) : bands;
        const int groups = shared ? 1 : (int)N;
        if (S <= 8) {
            dim3 grid((unsigned)((region + 255) / 256), (unsigned)(chunks * otiles), (unsigned)groups);
            hipLaunchKernelGGL(conv_dw_reduce_few_kernel, grid, dim3(256), 0, s, dw, partial, S, (int)C, (int)O, otiles,
                               (long)((size_t)S * region), (long)(C * 9 * O));
        } else {
            dim3 grid((unsigned)((region + 31) / 32), (unsigned)(chunks * otiles), (unsigned)groups);
            hipLaunchKernelGGL(conv_dw_reduce_kernel, grid, dim3(256), 0, s, dw, partial, S, (int)C, (int)O, otiles,
                               (long)((size_t)S * region), (long)(C * 9 * O));
        }
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) rc = set_hip_error(e, "conv_dw_reduce kernel launch");
    }
    int rc2 = workspace_free(partial, s);
    return rc ? rc : rc2;
}
