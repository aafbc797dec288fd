// Measurement hooks: what this GPU sustains when nothing but the matrix pipes, or nothing but the
// memory system, is at work. A benchmark reports a kernel against the published peaks and against these
// two figures; neither is part of any product path.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>

#include "nzhip_internal.h"

namespace nzhip {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// One wave per SIMD, the 64 accumulators of a 128 x 128 wave tile, eight A and eight B fragments held
// in registers; per pass 64 v_mfma_f32_16x16x32_f16 that walk the accumulators in ascending order (the
// order the GEMM kernels use). Lane 0 of every workgroup notes the shader clock counter and the
// constant-rate (100 MHz) counter before and after the loop: their ratio is the clock the chip held.
__global__ __launch_bounds__(256) void probe_mfma_kernel(const half8_t* __restrict__ src, float* __restrict__ sink,
                                                         unsigned long long* __restrict__ stamps, int passes) {
    const int lane = threadIdx.x & 63;
    half8_t a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        a[i] = src[i * 64 + lane];
        b[i] = src[(8 + i) * 64 + lane];
    }
    floatx4 acc[64];
#pragma unroll
    for (int t = 0; t < 64; t++) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
    unsigned long long c0 = 0, r0 = 0;
    if (threadIdx.x == 0) {
        c0 = __builtin_readcyclecounter();
        r0 = wall_clock64();
    }
    for (int it = 0; it < passes; it++) {
#pragma unroll
        for (int t = 0; t < 64; t++)
            asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[t]) : "v"(a[t >> 3]), "v"(b[t & 7]));
    }
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    if (threadIdx.x == 0 && stamps) {
        stamps[2 * blockIdx.x] = __builtin_readcyclecounter() - c0;
        stamps[2 * blockIdx.x + 1] = wall_clock64() - r0;
    }
    float s = 0.f;
#pragma unroll
    for (int t = 0; t < 64; t++) s += acc[t][0] + acc[t][1] + acc[t][2] + acc[t][3];
    if (s == 12345.678f) sink[0] = s;                           // keeps the loop alive; never true in practice
}

__global__ __launch_bounds__(256) void probe_fill_kernel(_Float16* __restrict__ dst, int n, int zero) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    unsigned x = (unsigned)i * 2654435761u + 12345u;            // a fixed pseudo-random pattern in [-0.05, 0.05)
    x ^= x >> 15; x *= 2246822519u; x ^= x >> 13;
    dst[i] = zero ? (_Float16)0.f : (_Float16)(((x & 0xFFFF) / 65536.0f - 0.5f) * 0.1f);
}

__global__ __launch_bounds__(256) void probe_copy_kernel(floatx4* __restrict__ dst, const floatx4* __restrict__ src, size_t n16) {
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

}  // namespace nzhip

using namespace nzhip;

extern "C" {

int nzhip_probe_mfma(int passes, int zero_operands, void* workspace, size_t workspace_bytes, void* stream) {
    const int cus = device_cu_count();
    const size_t need = NZHIP_PROBE_MFMA_WORKSPACE_BYTES;
    if (passes < 1 || !workspace || workspace_bytes < need || cus > 1024)
        return set_error(NZHIP_E_INVALID, "nzhip_probe_mfma: passes >= 1 and a workspace of NZHIP_PROBE_MFMA_WORKSPACE_BYTES are needed");
    if (reinterpret_cast<uintptr_t>(workspace) & 15) return set_error(NZHIP_E_INVALID, "nzhip_probe_mfma: workspace must be 16-byte aligned");
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    char* ws = static_cast<char*>(workspace);
    unsigned long long* stamps = reinterpret_cast<unsigned long long*>(ws);               // 2 x 1024 counters
    _Float16* frag = reinterpret_cast<_Float16*>(ws + 16384);                             // 16 fragments x 64 lanes x 8
    float* sink = reinterpret_cast<float*>(ws + 16384 + 16 * 64 * 8 * 2);
    hipLaunchKernelGGL(probe_fill_kernel, dim3(32), dim3(256), 0, s, frag, 16 * 64 * 8, zero_operands);
    hipLaunchKernelGGL(probe_mfma_kernel, dim3((unsigned)cus), dim3(256), 0, s, reinterpret_cast<const half8_t*>(frag), sink, stamps, passes);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? NZHIP_OK : set_hip_error(e, "probe_mfma_kernel launch");
}

int nzhip_probe_copy(void* dst, const void* src, size_t bytes, void* stream) {
    if (!dst || !src || (bytes & 15) || ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15))
        return set_error(NZHIP_E_INVALID, "nzhip_probe_copy: 16-byte aligned buffers and a multiple of 16 bytes are needed");
    if (bytes == 0) return NZHIP_OK;
    const size_t n16 = bytes / 16;
    const unsigned blocks = (unsigned)std::min<size_t>((n16 + 255) / 256, (size_t)device_cu_count() * 32);
    hipLaunchKernelGGL(probe_copy_kernel, dim3(blocks), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                       static_cast<floatx4*>(dst), static_cast<const floatx4*>(src), n16);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? NZHIP_OK : set_hip_error(e, "probe_copy_kernel launch");
}

}  // extern "C"
