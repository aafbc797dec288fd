// Runtime of libnzhip.so: error reporting, the device caching allocator and the stream
// manager. Replaces cuStrm::StreamManager<float> + EventPool of the reference
// (include/NeuZephyr/StreamManager.cuh:131-911, EventPool.cuh:165-457).
//
// Design: ONE ordered compute stream. The reference hands every op a different one of 16
// streams and then re-creates the order with per-buffer events plus a host callback per op;
// since batches, broadcasts and epilogues run inside single kernels here, there is nothing
// left to overlap, and stream order itself is the dependency tracker. Blocking happens only
// in nzhip_sync_ptr / nzhip_sync_all / nzhip_memcpy_d2h / nzhip_free.
#include <cstdarg>
#include <cstdio>
#include <atomic>
#include <cstring>
#include <map>
#include <mutex>
#include <new>
#include <utility>

#include "nz_pool_allocator.hpp"
#include "nzhip_internal.h"

namespace nzhip {

static thread_local char g_err[512] = "";

int set_error(int status, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return status;
}

int set_hip_error(hipError_t e, const char* what) {
    snprintf(g_err, sizeof(g_err), "%s: %s (hipError_t %d)", what, hipGetErrorString(e), (int)e);
    return (int)e;
}

struct HipBackend {
    int raw_alloc(void** p, size_t bytes) {
        hipError_t e = hipMalloc(p, bytes);
        if (e != hipSuccess) {
            (void)hipGetLastError();   // clear the sticky error so the retry path starts clean
            *p = nullptr;
        }
        return (int)e;
    }
    int raw_free(void* p) { return (int)hipFree(p); }
};

class Runtime {
public:
    static Runtime& instance() {
        static Runtime* rt = new Runtime();   // intentionally leaked: no teardown races at exit
        return *rt;
    }
    int ensure_stream() {
        std::call_once(once_, [this] {
            hipError_t e = hipStreamCreateWithFlags(&stream_, hipStreamNonBlocking);
            if (e != hipSuccess) {
                init_status_ = set_hip_error(e, "hipStreamCreateWithFlags");
                stream_ = nullptr;
            }
        });
        return init_status_;
    }
    hipStream_t stream() {
        ensure_stream();
        return stream_;
    }
    PoolAllocator<HipBackend>& pool() { return pool_; }

private:
    Runtime() = default;
    std::once_flag once_;
    int init_status_ = 0;
    hipStream_t stream_ = nullptr;
    PoolAllocator<HipBackend> pool_;
};

// ---- static scratch: the workspace of the entry point that allocates nothing -----------------
// One array per GPU, held from the moment the library is loaded until the process ends. In host code
// the array's name is only a stand-in for the symbol: the device address comes from
// hipGetSymbolAddress, once per device with that device current, and only that address is ever
// handed to kernels.
constexpr size_t STATIC_SCRATCH_BYTES = NZHIP_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

static int static_scratch_base(unsigned char** base) {
    static std::mutex mu;
    static unsigned char* per_device[64] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return set_hip_error(e, "hipGetDevice");
    if (dev < 0 || dev >= 64) return set_error(NZHIP_E_UNSUPPORTED, "static scratch: device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(mu);
    if (!per_device[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) return set_hip_error(e, "hipGetSymbolAddress(static scratch)");
        per_device[dev] = static_cast<unsigned char*>(p);
    }
    *base = per_device[dev];
    return NZHIP_OK;
}

// While a thread is inside nzhip_gemm_static its workspace requests are served from the current
// device's static scratch (bump allocation, nothing is ever returned) instead of the pool.
struct StaticArena {
    unsigned char* base = nullptr;
    size_t used = 0;
    bool active = false;
};
static thread_local StaticArena t_arena;

int workspace_alloc(void** ptr, size_t bytes, hipStream_t s) {
    if (t_arena.active) {
        const size_t at = (t_arena.used + 255) & ~(size_t)255;
        if (bytes > STATIC_SCRATCH_BYTES || at > STATIC_SCRATCH_BYTES - bytes)
            return set_error(NZHIP_E_UNSUPPORTED,
                             "nzhip_gemm_static: this product needs %zu bytes of workspace, the static scratch holds %zu",
                             at + bytes, STATIC_SCRATCH_BYTES);
        *ptr = t_arena.base + at;
        t_arena.used = at + bytes;
        return NZHIP_OK;
    }
    int rc = Runtime::instance().pool().allocate(ptr, bytes, reinterpret_cast<uintptr_t>(s));
    if (rc != 0) return set_error(NZHIP_E_NOMEM, "workspace allocation of %zu bytes failed (hipError_t %d)", bytes, rc);
    return NZHIP_OK;
}

int workspace_free(void* ptr, hipStream_t s) {
    if (t_arena.active) return NZHIP_OK;                      // the arena is reset by the next call
    return Runtime::instance().pool().free_async(ptr, reinterpret_cast<uintptr_t>(s)) == 0
               ? NZHIP_OK
               : set_error(NZHIP_E_INVALID, "workspace_free: unknown pointer");
}

// ---- prepared operand images ----------------------------------------------------------------------------------
}  // namespace nzhip

struct nzhip_prepared {
    std::mutex mu;
    void* image = nullptr;
    size_t bytes = 0;
    bool valid = false;
    uint64_t key[nzhip::PREPARED_KEY_WORDS] = {};
    uintptr_t stream_tag = 0;                       // pool tag the image was allocated under
    unsigned long long fills = 0;                   // how often an image was (re)built through this handle
};

namespace nzhip {

struct PreparedScope {
    nzhip_prepared* handle = nullptr;
    int kind = 0;
};
static thread_local PreparedScope t_prepared;

bool image_kept_by_caller(int kind) { return t_prepared.handle && t_prepared.kind == kind && !t_arena.active; }

int image_acquire(int kind, const uint64_t key[PREPARED_KEY_WORDS], size_t bytes, hipStream_t s, ImageLease* out) {
    nzhip_prepared* h = (t_prepared.handle && t_prepared.kind == kind && !t_arena.active) ? t_prepared.handle : nullptr;
    if (!h) {
        out->fill = true;
        out->persistent = false;
        return workspace_alloc(&out->ptr, bytes, s);
    }
    std::lock_guard<std::mutex> lock(h->mu);
    out->persistent = true;
    if (h->valid && h->bytes == bytes && memcmp(h->key, key, sizeof(h->key)) == 0) {
        out->ptr = h->image;
        out->fill = false;
        return NZHIP_OK;
    }
    if (h->image && h->bytes != bytes) {            // another operand or another route: start over
        Runtime::instance().pool().free_async(h->image, h->stream_tag);
        h->image = nullptr;
    }
    if (!h->image) {
        const int rc = Runtime::instance().pool().allocate(&h->image, bytes, reinterpret_cast<uintptr_t>(s));
        if (rc != 0) {
            h->image = nullptr;
            h->valid = false;
            return set_error(NZHIP_E_NOMEM, "prepared image of %zu bytes: allocation failed (hipError_t %d)", bytes, rc);
        }
        h->stream_tag = reinterpret_cast<uintptr_t>(s);
    }
    h->bytes = bytes;
    memcpy(h->key, key, sizeof(h->key));
    h->valid = false;                               // until the release says that the image was built
    out->ptr = h->image;
    out->fill = true;
    out->owner = h;
    return NZHIP_OK;
}

int image_release(const ImageLease& lease, hipStream_t s, bool enqueued) {
    if (!lease.ptr) return NZHIP_OK;
    if (!lease.persistent) return workspace_free(lease.ptr, s);
    if (lease.fill && lease.owner) {
        nzhip_prepared* h = static_cast<nzhip_prepared*>(lease.owner);
        std::lock_guard<std::mutex> lock(h->mu);
        if (enqueued && h->image == lease.ptr) {
            h->valid = true;
            h->fills++;
        }
    }
    return NZHIP_OK;
}

int device_cu_count() {
    static std::atomic<int> cached[64];                          // 0 = not queried yet
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int cus = cached[dev].load(std::memory_order_relaxed);
    if (cus == 0) {
        hipDeviceProp_t prop;
        cus = hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
        cached[dev].store(cus, std::memory_order_relaxed);
    }
    return cus;
}

int ensure_dynamic_lds(const void* kernel, int bytes, const char* what) {
    static std::mutex mu;
    static std::map<std::pair<int, const void*>, int> reached;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return set_hip_error(e, "hipGetDevice");
    std::lock_guard<std::mutex> lock(mu);
    int& cur = reached[{dev, kernel}];
    if (cur >= bytes) return NZHIP_OK;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) return set_hip_error(e, what);
    cur = bytes;
    return NZHIP_OK;
}

}  // namespace nzhip

using namespace nzhip;

extern "C" {

int nzhip_version(void) { return 100; }

const char* nzhip_last_error(void) { return g_err; }

int nzhip_device_info(int* cu_count, size_t* lds_bytes_per_cu, char* arch_name, size_t arch_name_len) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return set_hip_error(e, "hipGetDevice");
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return set_hip_error(e, "hipGetDeviceProperties");
    if (cu_count) *cu_count = prop.multiProcessorCount;
    if (lds_bytes_per_cu) *lds_bytes_per_cu = prop.maxSharedMemoryPerMultiProcessor;
    if (arch_name && arch_name_len) {
        strncpy(arch_name, prop.gcnArchName, arch_name_len - 1);
        arch_name[arch_name_len - 1] = '\0';
    }
    return NZHIP_OK;
}

void* nzhip_default_stream(void) { return Runtime::instance().stream(); }

int nzhip_malloc(void** ptr, size_t bytes) {
    if (!ptr) return set_error(NZHIP_E_INVALID, "nzhip_malloc: null out-pointer");
    Runtime& rt = Runtime::instance();
    if (int rc = rt.ensure_stream()) return rc;
    int rc = rt.pool().allocate(ptr, bytes, reinterpret_cast<uintptr_t>(rt.stream()));
    if (rc != 0) return set_error(NZHIP_E_NOMEM, "nzhip_malloc: %zu bytes: hipError_t %d", bytes, rc);
    return NZHIP_OK;
}

int nzhip_free_async(void* ptr) {
    Runtime& rt = Runtime::instance();
    if (rt.pool().free_async(ptr, reinterpret_cast<uintptr_t>(rt.stream())) != 0)
        return set_error(NZHIP_E_INVALID, "nzhip_free_async: pointer %p is not a live nzhip allocation", ptr);
    return NZHIP_OK;
}

int nzhip_free(void* ptr) {
    if (!ptr) return NZHIP_OK;
    Runtime& rt = Runtime::instance();
    hipError_t e = hipDeviceSynchronize();
    if (e != hipSuccess) return set_hip_error(e, "hipDeviceSynchronize");
    if (rt.pool().free_now(ptr) != 0)
        return set_error(NZHIP_E_INVALID, "nzhip_free: pointer %p is not a live nzhip allocation", ptr);
    return NZHIP_OK;
}

int nzhip_host_malloc(void** ptr, size_t bytes) {
    if (!ptr) return set_error(NZHIP_E_INVALID, "nzhip_host_malloc: null out-pointer");
    *ptr = nullptr;
    if (bytes == 0) return NZHIP_OK;
    if (int rc = Runtime::instance().ensure_stream()) return rc;
    // page-locked and mapped: the same address is valid on the host and in kernels
    hipError_t e = hipHostMalloc(ptr, bytes, hipHostMallocMapped | hipHostMallocPortable);
    if (e != hipSuccess) {
        *ptr = nullptr;
        return set_error(NZHIP_E_NOMEM, "nzhip_host_malloc: %zu bytes: hipError_t %d", bytes, (int)e);
    }
    return NZHIP_OK;
}

int nzhip_host_free(void* ptr) {
    if (!ptr) return NZHIP_OK;
    hipError_t e = hipStreamSynchronize(Runtime::instance().stream());     // kernels may still read or write it
    if (e != hipSuccess) return set_hip_error(e, "hipStreamSynchronize");
    e = hipHostFree(ptr);
    return e == hipSuccess ? NZHIP_OK : set_hip_error(e, "hipHostFree");
}

int nzhip_memset(void* ptr, int value, size_t bytes) {
    if (!ptr && bytes) return set_error(NZHIP_E_INVALID, "nzhip_memset: null pointer");
    // whole fp32 words of one byte value (clearing gradients, the usual case) go through the library's own fill kernel:
    // a kernel node like any other for a caller that records the stream, where a memset node is a kind of its own
    if (bytes % 4 == 0 && (reinterpret_cast<uintptr_t>(ptr) & 3) == 0) {
        const unsigned word = 0x01010101u * (unsigned)(value & 0xff);
        float as_float;
        memcpy(&as_float, &word, sizeof(as_float));
        if (bytes == 0) return NZHIP_OK;
        return nzhip_fill(static_cast<float*>(ptr), as_float, bytes / 4, Runtime::instance().stream());
    }
    hipError_t e = hipMemsetAsync(ptr, value, bytes, Runtime::instance().stream());
    return e == hipSuccess ? NZHIP_OK : set_hip_error(e, "hipMemsetAsync");
}

static int copy(void* dst, const void* src, size_t bytes, hipMemcpyKind kind, const char* what) {
    if ((!dst || !src) && bytes) return set_error(NZHIP_E_INVALID, "%s: null pointer", what);
    hipError_t e = hipMemcpyAsync(dst, src, bytes, kind, Runtime::instance().stream());
    return e == hipSuccess ? NZHIP_OK : set_hip_error(e, what);
}

int nzhip_memcpy_h2d(void* dst, const void* src, size_t bytes) {
    // Pageable host memory: the runtime stages the source before returning, so the caller's
    // buffer may be reused at once; the device-side copy stays ordered on the compute stream.
    return copy(dst, src, bytes, hipMemcpyHostToDevice, "nzhip_memcpy_h2d");
}

int nzhip_memcpy_d2d(void* dst, const void* src, size_t bytes) {
    return copy(dst, src, bytes, hipMemcpyDeviceToDevice, "nzhip_memcpy_d2d");
}

int nzhip_memcpy_d2h(void* dst, const void* src, size_t bytes) {
    int rc = copy(dst, src, bytes, hipMemcpyDeviceToHost, "nzhip_memcpy_d2h");
    if (rc) return rc;
    hipError_t e = hipStreamSynchronize(Runtime::instance().stream());
    if (e != hipSuccess) return set_hip_error(e, "hipStreamSynchronize");
    // the copy has been carried out; what may still be reported is a single-kernel product that ran out of polls
    return gemm_h16_coop_check(Runtime::instance().stream(), false);
}

int nzhip_sync_ptr(const void* ptr) {
    (void)ptr;   // everything that touches ptr is ahead of this point in the runtime's stream (see nzhip.h)
    hipError_t e = hipStreamSynchronize(Runtime::instance().stream());
    if (e != hipSuccess) return set_hip_error(e, "hipStreamSynchronize");
    return gemm_h16_coop_check(Runtime::instance().stream(), false);
}

int nzhip_stream_wait(void* stream) {
    Runtime& rt = Runtime::instance();
    if (int rc = rt.ensure_stream()) return rc;
    hipStream_t other = static_cast<hipStream_t>(stream);
    if (other == rt.stream()) return NZHIP_OK;
    hipEvent_t ev = nullptr;
    hipError_t e = hipEventCreateWithFlags(&ev, hipEventDisableTiming);
    if (e != hipSuccess) return set_hip_error(e, "hipEventCreateWithFlags");
    e = hipEventRecord(ev, other);
    if (e == hipSuccess) e = hipStreamWaitEvent(rt.stream(), ev, 0);
    const hipError_t e2 = hipEventDestroy(ev);          // released by the runtime once the event has completed
    if (e != hipSuccess) return set_hip_error(e, "nzhip_stream_wait");
    return e2 == hipSuccess ? NZHIP_OK : set_hip_error(e2, "hipEventDestroy");
}

int nzhip_sync_all(void) {
    hipError_t e = hipDeviceSynchronize();
    if (e != hipSuccess) return set_hip_error(e, "hipDeviceSynchronize");
    return gemm_h16_coop_check(nullptr, true);
}

int nzhip_prepared_create(nzhip_prepared** handle) {
    if (!handle) return set_error(NZHIP_E_INVALID, "nzhip_prepared_create: null pointer");
    *handle = new (std::nothrow) nzhip_prepared();
    return *handle ? NZHIP_OK : set_error(NZHIP_E_NOMEM, "nzhip_prepared_create: out of host memory");
}

int nzhip_prepared_invalidate(nzhip_prepared* handle) {
    if (!handle) return set_error(NZHIP_E_INVALID, "nzhip_prepared_invalidate: null handle");
    std::lock_guard<std::mutex> lock(handle->mu);
    handle->valid = false;
    return NZHIP_OK;
}

int nzhip_prepared_fills(const nzhip_prepared* handle, unsigned long long* count) {
    if (!handle || !count) return set_error(NZHIP_E_INVALID, "nzhip_prepared_fills: null argument");
    std::lock_guard<std::mutex> lock(const_cast<nzhip_prepared*>(handle)->mu);
    *count = handle->fills;
    return NZHIP_OK;
}

int nzhip_prepared_destroy(nzhip_prepared* handle) {
    if (!handle) return NZHIP_OK;
    int rc = NZHIP_OK;
    if (handle->image && Runtime::instance().pool().free_async(handle->image, handle->stream_tag) != 0)
        rc = set_error(NZHIP_E_INVALID, "nzhip_prepared_destroy: the image is not a pool allocation");
    delete handle;
    return rc;
}

int nzhip_gemm_prepared_b(const nzhip_gemm_desc* desc, nzhip_prepared* b_image, void* stream) {
    if (!b_image) return nzhip_gemm(desc, stream);
    t_prepared.handle = b_image;
    t_prepared.kind = PREPARED_GEMM_B;
    const int rc = nzhip_gemm(desc, stream);
    t_prepared = PreparedScope();
    return rc;
}

int nzhip_conv2d_forward_prepared(float* y, const float* x, const float* w_ref, const float* bias, size_t N, size_t C, size_t H,
                                  size_t W, size_t O, size_t K_h, size_t K_w, size_t stride, size_t pad, size_t w_batch,
                                  int64_t bias_stride_pixel, int64_t bias_stride_channel, int activation,
                                  nzhip_prepared* w_image, void* stream) {
    t_prepared.handle = w_image;
    t_prepared.kind = PREPARED_CONV_W;
    const int rc = nzhip_conv2d_forward(y, x, w_ref, bias, N, C, H, W, O, K_h, K_w, stride, pad, w_batch, bias_stride_pixel,
                                        bias_stride_channel, activation, stream);
    t_prepared = PreparedScope();
    return rc;
}

int nzhip_gemm_static(const nzhip_gemm_desc* desc, void* stream) {
    unsigned char* base = nullptr;
    if (int rc = static_scratch_base(&base)) return rc;
    t_arena.base = base;
    t_arena.used = 0;
    t_arena.active = true;
    const int rc = nzhip_gemm(desc, stream);
    t_arena.active = false;
    return rc;
}

size_t nzhip_static_scratch_bytes(void) { return STATIC_SCRATCH_BYTES; }

int nzhip_allocator_stats(size_t* bytes_in_use, size_t* bytes_cached, size_t* device_allocs) {
    const PoolStats s = Runtime::instance().pool().stats();
    if (bytes_in_use) *bytes_in_use = s.bytes_in_use;
    if (bytes_cached) *bytes_cached = s.bytes_cached;
    if (device_allocs) *device_allocs = s.device_allocs;
    return NZHIP_OK;
}

int nzhip_allocator_trim(void) {
    hipError_t e = hipDeviceSynchronize();
    if (e != hipSuccess) return set_hip_error(e, "hipDeviceSynchronize");
    Runtime::instance().pool().trim();
    return NZHIP_OK;
}

}  // extern "C"
