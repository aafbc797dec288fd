// What stands between the convolution / linear layers and a loss in the reference's own example
// network (README.md:62-90: Conv2d, ReLU, Conv2d, AvgPool2d, Linear, Softmax, BCELoss): average
// pooling and its gradient (AveragePoolingKernel / AveragePoolingBackwardKernel,
// src/OperationKernels.cu:1404-1486), the binary cross-entropy loss and its gradient
// (BinaryCrossEntropyKernel / BCEBackwardKernel, :648-700) and the batch expansion of a target
// (ExpandKernel / CompressKernel, :1282-1301). All of them are streams over memory.
#include <hip/hip_runtime.h>

#include "nzhip_internal.h"

namespace nzhip {

static inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

static int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? NZHIP_OK : set_hip_error(e, what);
}

struct PoolArgs {
    int pool, stride, pad;
    int H_in, W_in, H_out, W_out;
    int wblocks, wblocks_in;    // 256-column blocks per output row / per input row
    long planes;                // batches * channels
    int overwrite;              // backward: din = the sums instead of din += them (din's old contents are not read)
};

// One thread per output element: the window is summed row by row, left to right (the reference's
// loop order), and divided by the number of window cells inside the image.
// POOL: the window extent at compile time (0: p.pool); a window inside the image is then pool^2 loads and adds
// without a loop or a bounds test.
template <int POOL>
__global__ __launch_bounds__(256) void avgpool_kernel(float* __restrict__ out, const float* __restrict__ in,
                                                      const PoolArgs p, const int cw_log, const int wblocks) {
    // grid: x = (block of 256 >> cw_log output rows, block of 1 << cw_log columns), y and z = plane; nothing here divides
    // per thread. Narrow images get several rows per workgroup instead of a row of mostly idle lanes.
    const int h = (blockIdx.x / wblocks) * (256 >> cw_log) + (threadIdx.x >> cw_log);
    const int w = ((blockIdx.x % wblocks) << cw_log) + (threadIdx.x & ((1 << cw_log) - 1));
    const long plane = blockIdx.y + (long)gridDim.y * blockIdx.z;
    if (w >= p.W_out || h >= p.H_out || plane >= p.planes) return;
    const long idx = (plane * p.H_out + h) * p.W_out + w;
    const int h0 = h * p.stride - p.pad, w0 = w * p.stride - p.pad;
    const float* src = in + plane * p.H_in * p.W_in;
    float sum = 0.f;
    int count = 0;
    if (POOL && h0 >= 0 && h0 + POOL <= p.H_in && w0 >= 0 && w0 + POOL <= p.W_in) {
        const float* win = src + (long)h0 * p.W_in + w0;
        float v[POOL ? POOL * POOL : 1];
#pragma unroll
        for (int i = 0; i < POOL; i++)
#pragma unroll
            for (int j = 0; j < POOL; j++) v[i * POOL + j] = win[(long)i * p.W_in + j];
#pragma unroll
        for (int k = 0; k < POOL * POOL; k++) sum += v[k];
        count = POOL * POOL;
    } else {
        for (int i = 0; i < p.pool; i++) {
            const int hi = h0 + i;
            if (hi < 0 || hi >= p.H_in) continue;
            for (int j = 0; j < p.pool; j++) {
                const int wi = w0 + j;
                if (wi >= 0 && wi < p.W_in) {
                    sum += src[(long)hi * p.W_in + wi];
                    count++;
                }
            }
        }
    }
    out[idx] = count > 0 ? sum / (float)count : 0.f;
}

// Gradient in two steps. First every output element's share dout / divisor is computed once (the divisor is
// pool^2 without padding and the number of window cells inside the image with padding, :1451-1480); then one
// thread per INPUT element adds, in ascending (row, column) order of the output windows that cover it, those
// shares onto the value already there. That is the order in which a serial run of the reference's scatter loop
// reaches this element, so the result does not depend on scheduling (the reference's atomicAdd order does).
__global__ __launch_bounds__(256) void avgpool_share_kernel(float* __restrict__ share, const float* __restrict__ dout,
                                                            const PoolArgs p) {
    const int oh = blockIdx.x / p.wblocks, ow = (blockIdx.x % p.wblocks) * 256 + threadIdx.x;
    const long plane = blockIdx.y + (long)gridDim.y * blockIdx.z;
    if (ow >= p.W_out || plane >= p.planes) return;
    const long idx = (plane * p.H_out + oh) * p.W_out + ow;
    const int h0 = oh * p.stride - p.pad, w0 = ow * p.stride - p.pad;
    const int rows = min(h0 + p.pool, p.H_in) - max(h0, 0), cols = min(w0 + p.pool, p.W_in) - max(w0, 0);
    const float div = p.pad == 0 ? (float)(p.pool * p.pool) : (float)(rows * cols);
    share[idx] = dout[idx] / div;
}

__global__ __launch_bounds__(256) void avgpool_backward_kernel(float* __restrict__ din, const float* __restrict__ share,
                                                               const PoolArgs p) {
    // grid: x = (input row, 256-column block; wblocks_in blocks per row), y and z = plane
    const int h = blockIdx.x / p.wblocks_in, w = (blockIdx.x % p.wblocks_in) * 256 + threadIdx.x;
    const long plane = blockIdx.y + (long)gridDim.y * blockIdx.z;
    if (w >= p.W_in || plane >= p.planes) return;
    const long idx = (plane * p.H_in + h) * p.W_in + w;
    // windows with oh*stride - pad <= h <= oh*stride - pad + pool - 1. The row bounds are the same for the
    // whole workgroup; the column bounds divide in fp32, which is exact for these magnitudes (< 2^24).
    const int hp = h + p.pad, wp = w + p.pad;
    int oh_lo = hp - p.pool + 1 <= 0 ? 0 : (hp - p.pool + p.stride) / p.stride;
    int oh_hi = hp / p.stride;
    const float fs = (float)p.stride;
    int ow_lo = wp - p.pool + 1 <= 0 ? 0 : (int)((float)(wp - p.pool + p.stride) / fs);
    int ow_hi = (int)((float)wp / fs);
    if (oh_hi > p.H_out - 1) oh_hi = p.H_out - 1;
    if (ow_hi > p.W_out - 1) ow_hi = p.W_out - 1;
    const float* g = share + plane * p.H_out * p.W_out;
    float acc = p.overwrite ? 0.f : din[idx];
    for (int oh = oh_lo; oh <= oh_hi; oh++)
        for (int ow = ow_lo; ow <= ow_hi; ow++) acc += g[(long)oh * p.W_out + ow];
    din[idx] = acc;
}

// The same sums for four adjacent input columns per thread (rows of whole 16-byte pieces): the gradient row moves as
// 16-byte accesses, and a share that several of the four columns need is requested once. Every column still adds its
// shares in ascending (row, column) order of the windows.
// RMAX, CMAX: the most window rows that cover an input row ((pool - 1) / stride + 1) and the most window columns that
// cover four adjacent input columns ((pool + 2) / stride + 1), at compile time: all RMAX * CMAX shares are then requested
// at once (clamped addresses) before the first is added. 0: bounds known only at run time, one request per loop step.
template <int RMAX, int CMAX>
// This kernel reads dout and divides by the window's cell count itself (the same fp32 division as avgpool_share_kernel:
// a dozen divisions per thread cost less than a pass that writes the shares and another that reads them).
__global__ __launch_bounds__(256) void avgpool_backward_vec_kernel(float* __restrict__ din, const float* __restrict__ dout,
                                                                   const PoolArgs p, const int cw_log, const int wblocks4) {
    typedef float floatx4 __attribute__((ext_vector_type(4)));
    // (block of 256 >> cw_log input rows, block of 1 << cw_log column quads), as in the forward kernel
    const int h = (blockIdx.x / wblocks4) * (256 >> cw_log) + (threadIdx.x >> cw_log);
    const int w = (((blockIdx.x % wblocks4) << cw_log) + (threadIdx.x & ((1 << cw_log) - 1))) * 4;
    const long plane = blockIdx.y + (long)gridDim.y * blockIdx.z;
    if (w >= p.W_in || h >= p.H_in || plane >= p.planes) return;
    const long idx = (plane * p.H_in + h) * p.W_in + w;
    const int hp = h + p.pad;
    const int oh_lo = hp - p.pool + 1 <= 0 ? 0 : (hp - p.pool + p.stride) / p.stride;
    int oh_hi = hp / p.stride;
    if (oh_hi > p.H_out - 1) oh_hi = p.H_out - 1;
    const float fs = (float)p.stride;
    int lo[4], hi[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const int wp = w + e + p.pad;
        lo[e] = wp - p.pool + 1 <= 0 ? 0 : (int)((float)(wp - p.pool + p.stride) / fs);
        hi[e] = (int)((float)wp / fs);
        if (hi[e] > p.W_out - 1) hi[e] = p.W_out - 1;
    }
    const float* g = dout + plane * p.H_out * p.W_out;
    auto divisor = [&](const int oh, const int ow) {
        if (p.pad == 0) return (float)(p.pool * p.pool);
        const int h0 = oh * p.stride - p.pad, w0 = ow * p.stride - p.pad;
        const int rows = min(h0 + p.pool, p.H_in) - max(h0, 0), cols = min(w0 + p.pool, p.W_in) - max(w0, 0);
        return (float)(rows * cols);
    };
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
    if (!p.overwrite) acc = *reinterpret_cast<const floatx4*>(din + idx);
    if (RMAX) {
        float sv[RMAX ? RMAX * CMAX : 1];
#pragma unroll
        for (int r = 0; r < RMAX; r++)
#pragma unroll
            for (int c = 0; c < CMAX; c++) {
                const int oh = oh_lo + r, ow = lo[0] + c;
                const bool ok = oh <= oh_hi && ow <= hi[3];
                sv[r * CMAX + c] = g[ok ? (long)oh * p.W_out + ow : 0];
            }
#pragma unroll
        for (int r = 0; r < RMAX; r++)
#pragma unroll
            for (int c = 0; c < CMAX; c++) {
                const int oh = oh_lo + r, ow = lo[0] + c;
                const float v = sv[r * CMAX + c] / divisor(oh, ow);
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (oh <= oh_hi && ow >= lo[e] && ow <= hi[e]) acc[e] += v;
            }
    } else {
        for (int oh = oh_lo; oh <= oh_hi; oh++) {
            const float* grow = g + (long)oh * p.W_out;
            for (int ow = lo[0]; ow <= hi[3]; ow++) {                   // (bounds are monotone in the column)
                const float v = grow[ow] / divisor(oh, ow);
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (ow >= lo[e] && ow <= hi[e]) acc[e] += v;
            }
        }
    }
    *reinterpret_cast<floatx4*>(din + idx) = acc;
}

// ---- binary cross-entropy ------------------------------------------------------------------------
// loss = sum_i (-t_i log p_i - (1 - t_i) log(1 - p_i)) / n. Two steps with a fixed shape: up to 1024
// workgroups add their grid-strided terms (lane, wave shuffle, four waves), then one workgroup adds the
// partial sums the same way, so the value depends on n only. __logf is the fast hardware logarithm,
// as in the reference's kernel.
constexpr int BCE_MAX_BLOCKS = 1024;

__device__ __forceinline__ float block_sum_256(float v, float* part) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = v;
    __syncthreads();
    return (part[0] + part[1]) + (part[2] + part[3]);
}

__global__ __launch_bounds__(256) void bce_partial_kernel(float* __restrict__ partial, const float* __restrict__ predict,
                                                          const float* __restrict__ real, long n) {
    __shared__ float part[4];
    float s = 0.f;
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
        const float p = predict[i], t = real[i];
        s += (-t * __logf(p) - (1 - t) * __logf(1 - p)) / (float)n;
    }
    const float total = block_sum_256(s, part);
    if (threadIdx.x == 0) partial[blockIdx.x] = total;
}

// Mean squared error with the same two-step summation: sum_i (p_i - t_i)^2 / n (MeanSquaredErrorKernel, :579-619).
__global__ __launch_bounds__(256) void mse_partial_kernel(float* __restrict__ partial, const float* __restrict__ predict,
                                                          const float* __restrict__ real, long n) {
    __shared__ float part[4];
    float s = 0.f;
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
        const float d = predict[i] - real[i];
        s += d * d / (float)n;
    }
    const float total = block_sum_256(s, part);
    if (threadIdx.x == 0) partial[blockIdx.x] = total;
}

__global__ __launch_bounds__(256) void mse_backward_kernel(float* __restrict__ grad, const float* __restrict__ predict,
                                                           const float* __restrict__ real, long n) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i < n) grad[i] = 2 * (predict[i] - real[i]) / (float)n;
}

__global__ __launch_bounds__(256) void bce_final_kernel(float* __restrict__ loss, const float* __restrict__ partial, int m) {
    __shared__ float part[4];
    float s = 0.f;
    for (int i = threadIdx.x; i < m; i += 256) s += partial[i];
    const float total = block_sum_256(s, part);
    if (threadIdx.x == 0) *loss = total;
}

__global__ __launch_bounds__(256) void bce_backward_kernel(float* __restrict__ grad, const float* __restrict__ predict,
                                                           const float* __restrict__ real, long n) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float p = predict[i];
    grad[i] = ((p - real[i]) / (p * (1 - p))) / (float)n;
}

// ---- expand / compress --------------------------------------------------------------------------
__global__ __launch_bounds__(256) void expand_kernel(float* __restrict__ out, const float* __restrict__ in, long n, long total) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i < total) out[i] = in[i % n];
}

// out[j] += in[j] + in[n + j] + ... in ascending batch order (a serial run of the reference's atomicAdd loop)
__global__ __launch_bounds__(256) void compress_kernel(float* __restrict__ out, const float* __restrict__ in, long n, long batches) {
    const long j = (long)blockIdx.x * 256 + threadIdx.x;
    if (j >= n) return;
    float acc = out[j];
    for (long b = 0; b < batches; b++) acc += in[b * n + j];
    out[j] = acc;
}

static int pool_args(PoolArgs& p, size_t pool, size_t stride, size_t pad, size_t batches, size_t channels, size_t H_in,
                     size_t W_in, size_t H_out, size_t W_out, const char* who) {
    if (pool == 0 || stride == 0) return set_error(NZHIP_E_INVALID, "%s: zero pool size or stride", who);
    if (H_in + 2 * pad < pool || W_in + 2 * pad < pool) return set_error(NZHIP_E_SHAPE, "%s: window larger than the padded input", who);
    if (H_out != (H_in + 2 * pad - pool) / stride + 1 || W_out != (W_in + 2 * pad - pool) / stride + 1)
        return set_error(NZHIP_E_SHAPE, "%s: output extent does not match (in + 2 pad - pool) / stride + 1", who);
    if (pool > 0x7fff || stride > 0x3fffffff || pad > 0x3fffffff || H_in > 0x3fffffff || W_in > 0x3fffffff ||
        batches * channels > 0x7fffffffffffull / ((H_in * W_in) | 1))
        return set_error(NZHIP_E_UNSUPPORTED, "%s: extent too large", who);
    p.pool = (int)pool; p.stride = (int)stride; p.pad = (int)pad;
    p.H_in = (int)H_in; p.W_in = (int)W_in; p.H_out = (int)H_out; p.W_out = (int)W_out;
    p.planes = (long)(batches * channels);
    p.overwrite = 0;
    p.wblocks = (int)((W_out + 255) / 256);
    p.wblocks_in = (int)((W_in + 255) / 256);
    if (W_in + pad + stride >= (1u << 24) || (size_t)p.wblocks_in * H_in > 0x7fffffffull ||
        (size_t)p.wblocks * H_out > 0x7fffffffull || batches * channels > 65535ull * 65535ull)
        return set_error(NZHIP_E_UNSUPPORTED, "%s: extent too large", who);
    return NZHIP_OK;
}

// log2 of the column-block width for rows of `width` elements: the power of two from 16 to 256 that covers them
static int pool_cw_log(long width) {
    int cw_log = 8;
    while (cw_log > 4 && (1l << (cw_log - 1)) >= width) cw_log--;
    return cw_log;
}

// x = rows x column blocks, planes folded into y (up to 65535) and z
static dim3 pool_grid(int wblocks, int rows, long planes) {
    const long gy = planes < 65535 ? planes : 65535;
    return dim3((unsigned)((long)wblocks * rows), (unsigned)gy, (unsigned)((planes + gy - 1) / gy));
}

}  // namespace nzhip

using namespace nzhip;

extern "C" {

int nzhip_avgpool2d(float* out, const float* in, size_t pool, size_t stride, size_t pad, size_t batches, size_t channels,
                    size_t H_in, size_t W_in, size_t H_out, size_t W_out, void* stream) {
    if (!out || !in) return set_error(NZHIP_E_INVALID, "nzhip_avgpool2d: null pointer");
    PoolArgs p;
    if (int rc = pool_args(p, pool, stride, pad, batches, channels, H_in, W_in, H_out, W_out, "nzhip_avgpool2d")) return rc;
    const size_t total = batches * channels * H_out * W_out;
    if (total == 0) return NZHIP_OK;
    auto kfn = p.pool == 2 ? avgpool_kernel<2> : p.pool == 3 ? avgpool_kernel<3> : p.pool == 5 ? avgpool_kernel<5> : avgpool_kernel<0>;
    const int cw_log = pool_cw_log(p.W_out), wblocks = (p.W_out + (1 << cw_log) - 1) >> cw_log, rb = 256 >> cw_log;
    hipLaunchKernelGGL(kfn, pool_grid(wblocks, (p.H_out + rb - 1) / rb, p.planes), dim3(256), 0, as_stream(stream), out, in, p, cw_log, wblocks);
    return check_launch("avgpool_kernel");
}

static int avgpool2d_backward_impl(float* din, const float* dout, size_t pool, size_t stride, size_t pad, size_t batches, size_t channels,
                                   size_t H_in, size_t W_in, size_t H_out, size_t W_out, int overwrite, void* stream);
int nzhip_avgpool2d_backward(float* din, const float* dout, size_t pool, size_t stride, size_t pad, size_t batches,
                             size_t channels, size_t H_in, size_t W_in, size_t H_out, size_t W_out, void* stream) {
    return avgpool2d_backward_impl(din, dout, pool, stride, pad, batches, channels, H_in, W_in, H_out, W_out, 0, stream);
}
int nzhip_avgpool2d_backward_overwrite(float* din, const float* dout, size_t pool, size_t stride, size_t pad, size_t batches,
                                       size_t channels, size_t H_in, size_t W_in, size_t H_out, size_t W_out, void* stream) {
    return avgpool2d_backward_impl(din, dout, pool, stride, pad, batches, channels, H_in, W_in, H_out, W_out, 1, stream);
}
static int avgpool2d_backward_impl(float* din, const float* dout, size_t pool, size_t stride, size_t pad, size_t batches, size_t channels,
                                   size_t H_in, size_t W_in, size_t H_out, size_t W_out, int overwrite, void* stream) {
    if (!din || !dout) return set_error(NZHIP_E_INVALID, "nzhip_avgpool2d_backward: null pointer");
    PoolArgs p;
    if (int rc = pool_args(p, pool, stride, pad, batches, channels, H_in, W_in, H_out, W_out, "nzhip_avgpool2d_backward")) return rc;
    p.overwrite = overwrite;
    const size_t total = batches * channels * H_in * W_in;
    if (total == 0) return NZHIP_OK;
    const size_t outs = batches * channels * H_out * W_out;
    if (outs == 0) return overwrite ? nzhip_fill(din, 0.f, total, stream) : NZHIP_OK;      // no window at all: the gradient is zero
    hipStream_t s = as_stream(stream);
    if (p.W_in % 4 == 0 && (reinterpret_cast<uintptr_t>(din) & 15) == 0) {
        const int cw_log = pool_cw_log(p.W_in / 4), wblocks4 = (p.W_in / 4 + (1 << cw_log) - 1) >> cw_log, rb = 256 >> cw_log;
        const int rmax = (p.pool - 1) / p.stride + 1, cmax = (p.pool + 2) / p.stride + 1;
        auto kfn = rmax == 3 && cmax == 4   ? avgpool_backward_vec_kernel<3, 4>      // 5 / 2
                   : rmax == 2 && cmax == 3 ? avgpool_backward_vec_kernel<2, 3>      // 3 / 2
                   : rmax == 1 && cmax == 3 ? avgpool_backward_vec_kernel<1, 3>      // 2 / 2
                   : rmax == 3 && cmax == 6 ? avgpool_backward_vec_kernel<3, 6>      // 3 / 1
                   : rmax == 2 && cmax == 5 ? avgpool_backward_vec_kernel<2, 5>      // 2 / 1
                                            : avgpool_backward_vec_kernel<0, 0>;
        hipLaunchKernelGGL(kfn, pool_grid(wblocks4, (p.H_in + rb - 1) / rb, p.planes), dim3(256), 0, s, din, dout, p, cw_log, wblocks4);
        return check_launch("avgpool_backward_vec_kernel");
    }
    float* share = nullptr;
    if (int rc = workspace_alloc(reinterpret_cast<void**>(&share), outs * sizeof(float), s)) return rc;
    hipLaunchKernelGGL(avgpool_share_kernel, pool_grid(p.wblocks, p.H_out, p.planes), dim3(256), 0, s, share, dout, p);
    int rc = check_launch("avgpool_share_kernel");
    if (rc == NZHIP_OK) {
        hipLaunchKernelGGL(avgpool_backward_kernel, pool_grid(p.wblocks_in, p.H_in, p.planes), dim3(256), 0, s, din, share, p);
        rc = check_launch("avgpool_backward_kernel");
    }
    const int rc2 = workspace_free(share, s);
    return rc ? rc : rc2;
}

static int mean_loss(float* loss, const float* predict, const float* real, size_t n, void* stream, bool bce, const char* who) {
    if (!loss || ((!predict || !real) && n)) return set_error(NZHIP_E_INVALID, "%s: null pointer", who);
    hipStream_t s = as_stream(stream);
    size_t blocks = (n + 255) / 256;
    if (blocks > (size_t)BCE_MAX_BLOCKS) blocks = BCE_MAX_BLOCKS;
    if (blocks == 0) blocks = 1;                                  // n = 0: the sum of nothing
    float* partial = nullptr;
    if (int rc = workspace_alloc(reinterpret_cast<void**>(&partial), blocks * sizeof(float), s)) return rc;
    if (bce) hipLaunchKernelGGL(bce_partial_kernel, dim3((unsigned)blocks), dim3(256), 0, s, partial, predict, real, (long)n);
    else hipLaunchKernelGGL(mse_partial_kernel, dim3((unsigned)blocks), dim3(256), 0, s, partial, predict, real, (long)n);
    int rc = check_launch("loss partial kernel");
    if (rc == NZHIP_OK) {
        hipLaunchKernelGGL(bce_final_kernel, dim3(1), dim3(256), 0, s, loss, partial, (int)blocks);
        rc = check_launch("bce_final_kernel");
    }
    const int rc2 = workspace_free(partial, s);
    return rc ? rc : rc2;
}

int nzhip_bce_loss(float* loss, const float* predict, const float* real, size_t n, void* stream) {
    return mean_loss(loss, predict, real, n, stream, true, "nzhip_bce_loss");
}

int nzhip_mse_loss(float* loss, const float* predict, const float* real, size_t n, void* stream) {
    return mean_loss(loss, predict, real, n, stream, false, "nzhip_mse_loss");
}

int nzhip_mse_backward(float* grad, const float* predict, const float* real, size_t n, void* stream) {
    if ((!grad || !predict || !real) && n) return set_error(NZHIP_E_INVALID, "nzhip_mse_backward: null pointer");
    if (n == 0) return NZHIP_OK;
    if ((n + 255) / 256 > 0x7fffffffull) return set_error(NZHIP_E_UNSUPPORTED, "nzhip_mse_backward: extent too large");
    hipLaunchKernelGGL(mse_backward_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, as_stream(stream), grad, predict,
                       real, (long)n);
    return check_launch("mse_backward_kernel");
}

int nzhip_bce_backward(float* grad, const float* predict, const float* real, size_t n, void* stream) {
    if ((!grad || !predict || !real) && n) return set_error(NZHIP_E_INVALID, "nzhip_bce_backward: null pointer");
    if (n == 0) return NZHIP_OK;
    if ((n + 255) / 256 > 0x7fffffffull) return set_error(NZHIP_E_UNSUPPORTED, "nzhip_bce_backward: extent too large");
    hipLaunchKernelGGL(bce_backward_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, as_stream(stream), grad, predict,
                       real, (long)n);
    return check_launch("bce_backward_kernel");
}

int nzhip_expand(float* out, const float* in, size_t n, size_t batches, void* stream) {
    if ((!out || !in) && n * batches) return set_error(NZHIP_E_INVALID, "nzhip_expand: null pointer");
    const size_t total = n * batches;
    if (total == 0) return NZHIP_OK;
    if ((total + 255) / 256 > 0x7fffffffull) return set_error(NZHIP_E_UNSUPPORTED, "nzhip_expand: extent too large");
    hipLaunchKernelGGL(expand_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, as_stream(stream), out, in, (long)n,
                       (long)total);
    return check_launch("expand_kernel");
}

int nzhip_compress(float* out, const float* in, size_t n, size_t batches, void* stream) {
    if ((!out || !in) && n * batches) return set_error(NZHIP_E_INVALID, "nzhip_compress: null pointer");
    if (n == 0 || batches == 0) return NZHIP_OK;
    if ((n + 255) / 256 > 0x7fffffffull) return set_error(NZHIP_E_UNSUPPORTED, "nzhip_compress: extent too large");
    hipLaunchKernelGGL(compress_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, as_stream(stream), out, in, (long)n,
                       (long)batches);
    return check_launch("compress_kernel");
}

}  // extern "C"
