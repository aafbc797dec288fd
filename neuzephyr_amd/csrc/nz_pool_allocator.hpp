// Caching device allocator, independent of the GPU runtime: the Backend policy supplies
// raw_alloc/raw_free, so the bookkeeping can be unit-tested (and run under sanitizers) on a
// host without a GPU.
//
// Replaces the cudaMallocAsync / cudaFreeAsync pair behind the reference's
// StreamManager::malloc / freeAsync (include/NeuZephyr/StreamManager.cuh:230-240, 325-335).
// Semantics kept: allocation and release are ordered with a stream, so a block released by
// free_async may be handed out again immediately to later work on THAT stream. Blocks are
// therefore cached per stream tag and never migrate between streams while cached.
// Not kept: the reference multiplies a byte count by sizeof(T) a second time (4x
// over-allocation); sizes here are plain bytes.
#ifndef NZ_POOL_ALLOCATOR_HPP
#define NZ_POOL_ALLOCATOR_HPP

#include <cstddef>
#include <cstdint>
#include <map>
#include <mutex>
#include <unordered_map>

namespace nzhip {

struct PoolStats {
    size_t bytes_in_use = 0;    // rounded bytes currently handed out
    size_t bytes_cached = 0;    // rounded bytes sitting in free lists
    size_t device_allocs = 0;   // raw_alloc calls that succeeded
    size_t device_frees = 0;
    size_t cache_hits = 0;
};

// Size classes: multiples of 512 B below 1 MiB, multiples of 2 MiB above (HBM page
// granularity); a cached block serves a request when it is at most 25 % larger.
inline size_t pool_round_size(size_t bytes) {
    if (bytes == 0) bytes = 1;
    constexpr size_t kSmall = 512, kLarge = size_t(2) << 20, kSplit = size_t(1) << 20;
    const size_t q = bytes < kSplit ? kSmall : kLarge;
    return (bytes + q - 1) / q * q;
}

template <class Backend>
class PoolAllocator {
public:
    explicit PoolAllocator(Backend backend = Backend()) : backend_(backend) {}
    ~PoolAllocator() { trim(); }
    PoolAllocator(const PoolAllocator&) = delete;
    PoolAllocator& operator=(const PoolAllocator&) = delete;

    // 0 on success; otherwise the backend's error code (and *out = nullptr).
    int allocate(void** out, size_t bytes, uintptr_t stream_tag = 0) {
        if (!out) return -1;
        const size_t want = pool_round_size(bytes);
        std::lock_guard<std::mutex> lock(mu_);
        auto it = free_.lower_bound(Key{stream_tag, want});
        if (it != free_.end() && it->first.tag == stream_tag && it->first.size <= want + want / 4) {
            void* p = it->second;
            const size_t sz = it->first.size;
            free_.erase(it);
            live_[p] = sz;
            stats_.bytes_cached -= sz;
            stats_.bytes_in_use += sz;
            stats_.cache_hits++;
            *out = p;
            return 0;
        }
        void* p = nullptr;
        int rc = backend_.raw_alloc(&p, want);
        if (rc != 0) {
            // Out of device memory: give cached blocks back and retry once.
            release_cached_locked();
            rc = backend_.raw_alloc(&p, want);
            if (rc != 0) {
                *out = nullptr;
                return rc;
            }
        }
        live_[p] = want;
        stats_.bytes_in_use += want;
        stats_.device_allocs++;
        *out = p;
        return 0;
    }

    // Stream-ordered release: the block becomes reusable by later allocations at once.
    // Returns -1 for a pointer this allocator does not own (or a double free).
    int free_async(void* p, uintptr_t stream_tag = 0) {
        if (!p) return 0;
        std::lock_guard<std::mutex> lock(mu_);
        auto it = live_.find(p);
        if (it == live_.end()) return -1;
        const size_t sz = it->second;
        live_.erase(it);
        free_.emplace(Key{stream_tag, sz}, p);
        stats_.bytes_in_use -= sz;
        stats_.bytes_cached += sz;
        return 0;
    }

    // Immediate release to the backend (caller has synchronised).
    int free_now(void* p) {
        if (!p) return 0;
        std::lock_guard<std::mutex> lock(mu_);
        auto it = live_.find(p);
        if (it == live_.end()) return -1;
        stats_.bytes_in_use -= it->second;
        live_.erase(it);
        stats_.device_frees++;
        return backend_.raw_free(p);
    }

    bool owns(const void* p) const {
        std::lock_guard<std::mutex> lock(mu_);
        return live_.count(const_cast<void*>(p)) != 0;
    }

    void trim() {
        std::lock_guard<std::mutex> lock(mu_);
        release_cached_locked();
    }

    PoolStats stats() const {
        std::lock_guard<std::mutex> lock(mu_);
        return stats_;
    }

private:
    void release_cached_locked() {
        for (auto& kv : free_) {
            backend_.raw_free(kv.second);
            stats_.device_frees++;
        }
        free_.clear();
        stats_.bytes_cached = 0;
    }

    Backend backend_;
    mutable std::mutex mu_;
    struct Key {
        uintptr_t tag;
        size_t size;
        bool operator<(const Key& o) const { return tag != o.tag ? tag < o.tag : size < o.size; }
    };
    std::multimap<Key, void*> free_;
    std::unordered_map<void*, size_t> live_;
    PoolStats stats_;
};

}  // namespace nzhip

#endif
