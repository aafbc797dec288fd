// Internal declarations shared by the translation units of libnzhip.so.
#ifndef NZHIP_INTERNAL_H
#define NZHIP_INTERNAL_H

#include <hip/hip_runtime.h>

#include <cstdint>

#include "../../include/nzhip.h"

namespace nzhip {

// Record a failure for nzhip_last_error() and return the status to hand to the caller.
int set_error(int status, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int set_hip_error(hipError_t e, const char* what);

// MFMA tile kernels (nzhip_gemm.hip). force_tile: 0 = choose, 128 / 256 = that square tile.
// k_total > 0: the inner batch members are consecutive chunks of one contraction of that length
// (d.K is the chunk length; the last member contracts what is left)
int gemm_mfma_dispatch(const nzhip_gemm_desc& d, hipStream_t stream, int force_tile, int64_t k_total = 0, int padded = 0);
// Tile (64 or 128) and number of contraction chunks (1 = no split) for a product that goes to the fused kernel.
struct GemmPlan { int tile; int64_t parts; int64_t Kc; double cost_us; };
GemmPlan gemm_fused_plan(const nzhip_gemm_desc& d, int padded = 0);
bool gemm_small_tile(const nzhip_gemm_desc& d, int padded = 0);
// Two-pass route for large products: fp16 rounding pass + fp16 GEMM fed by direct-to-LDS loads
// (nzhip_gemm_h16.hip).
bool gemm_h16_applicable(const nzhip_gemm_desc& d);
bool gemm_vec_legal(const nzhip_gemm_desc& d);   // 16-byte global accesses are legal for A, B and C
bool gemm_operand_vec_legal(const float* X, int64_t ld, int64_t contig, int64_t stride_n, int64_t stride_c);
bool gemm_operands_vec_legal(const nzhip_gemm_desc& d, int padded = 0);   // ... for A and B (decides the kernel instance)
bool gemm_c_vec_legal(const nzhip_gemm_desc& d);          // ... for C (decides the epilogue's stores)
// nzhip_gemm for operands the library itself made: padded bit 0 / bit 1 = the rows of A / B are readable up to the next
// multiple of 4 elements and hold zeros there, so 16-byte loads are legal although the extents are not multiples of 4.
int gemm_padded_rows(const nzhip_gemm_desc& d, int padded, hipStream_t stream);
// waves: 0 = choose, else 2 / 4 / 8; mfma: 0 = choose, else 16 (16x16x32) / 32 (32x32x16)
int gemm_h16_dispatch(const nzhip_gemm_desc& d, hipStream_t stream, int waves = 0, int mfma = 0);
// Both passes in one kernel (rounding overlapped with the MFMA loop) for products of whole 4096 x 4096 x 1024 blocks.
bool gemm_h16_coop_applicable(const nzhip_gemm_desc& d);
int gemm_h16_coop_dispatch(const nzhip_gemm_desc& d, hipStream_t stream);
// After `drained` (or, with whole_device, every stream) has been synchronised: NZHIP_E_TIMEOUT once if a
// single-kernel product that has finished by now ran out of polls; the route is switched off from then on.
int gemm_h16_coop_check(hipStream_t drained, bool whole_device);
int gemm_h16_coop_reset(unsigned inject);
void gemm_h16_coop_test_mode(unsigned spin_limit, int mute);   // test hook: bound of the waits (0 = default), producers that do not signal
int gemm_h16_coop_timeouts(unsigned* count);     // polls that gave up since the library was loaded (expected: 0)
// Bandwidth-bound kernels for M <= 8 (nzhip_skinny.hip).
int gemm_skinny_dispatch(const nzhip_gemm_desc& d, hipStream_t stream);
bool gemm_skinny_applicable(const nzhip_gemm_desc& d);
// short contraction (K <= 32), one extent <= 16, the other long: streamed, one lane per long index
bool gemm_thin_applicable(const nzhip_gemm_desc& d);
int gemm_thin_dispatch(const nzhip_gemm_desc& d, hipStream_t stream);

// Stream-ordered workspace from the caching allocator (nzhip_runtime.cpp).
int workspace_alloc(void** ptr, size_t bytes, hipStream_t stream);
int workspace_free(void* ptr, hipStream_t stream);

// ---- prepared operand images (nzhip_prepared) -------------------------------------------------------------
// A kernel route that first turns an operand into an fp16 image (the two-pass GEMM's B image, the conv kernels'
// weight images) asks image_acquire() for the memory instead of workspace_alloc(). Outside a *_prepared entry
// point that is a pooled workspace and *fill is always true. Inside one (the calling thread carries the handle),
// the memory belongs to the handle: when the handle already holds an image built from the same key (operand
// address, extents, image kind) *fill comes back false and the conversion kernel is skipped.
// kind: which entry point the site belongs to; a handle is only honoured by sites of the kind it was passed for.
constexpr int PREPARED_GEMM_B = 1, PREPARED_CONV_W = 2;
constexpr int PREPARED_KEY_WORDS = 12;
struct ImageLease {
    void* ptr = nullptr;
    bool fill = true;           // the caller must (re)build the image
    bool persistent = false;    // owned by a handle: image_release leaves the memory alone
    void* owner = nullptr;      // that handle
};
int image_acquire(int kind, const uint64_t key[PREPARED_KEY_WORDS], size_t bytes, hipStream_t s, ImageLease* out);
// True while a *_prepared entry point of this kind is on the calling thread's stack with a handle: an image built now is kept.
bool image_kept_by_caller(int kind);
// `enqueued`: every launch between acquire and release went through. A handle whose image was to be rebuilt under this
// lease is only then marked as holding it; otherwise the next call rebuilds.
int image_release(const ImageLease& lease, hipStream_t s, bool enqueued);

// Compute units of the current device (queried once per device, then cached).
int device_cu_count();

// Raise a kernel's dynamic LDS limit to at least `bytes` on the current device. The limit reached is
// remembered per (device, kernel), so repeated launches cost a table lookup, not a driver call.
int ensure_dynamic_lds(const void* kernel, int bytes, const char* what);

}  // namespace nzhip

#endif
