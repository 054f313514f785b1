// Caching device-buffer pool: hipMalloc-backed, never zero-fills, recycles freed blocks by size
// class. The device-side counterpart of the host `Vec` recycling in
// crates/ft-core/src/buffer_pool.rs:206-329 and of `build_uninit`
// (crates/ft-kernel-cpu/src/lib.rs:2611-2639).
#pragma once

#include <cstddef>
#include <cstdint>

namespace fth {

// Returns FTH_OK and a device pointer of at least `bytes` bytes (NULL for 0 bytes).
int32_t pool_alloc(void **dptr, size_t bytes);
// Gives the block back for reuse. The caller guarantees that every kernel reading or writing it
// has completed or is ordered before the next user on the library's stream.
void pool_free(void *dptr);
void pool_stats(uint64_t *in_use, uint64_t *cached);
int32_t pool_trim();

// Frees every tracked block on scope exit.
class Scratch {
   public:
    Scratch() = default;
    Scratch(const Scratch &) = delete;
    Scratch &operator=(const Scratch &) = delete;
    ~Scratch();
    // Allocates `bytes` from the pool and tracks it.
    int32_t get(void **dptr, size_t bytes);

   private:
    static constexpr int kMax = 16;
    void *ptrs_[kMax] = {};
    int n_ = 0;
};

}  // namespace fth
