// The pool's backing store on a real device: plain hipMalloc / hipFree.
#pragma once

#include <mutex>
#include <unordered_map>

#include "pool.h"
#include "side_map.h"

namespace sideaware {

class HipBacking final : public Backing {
public:
    explicit HipBacking(int device) : device_(device), sides_(device) {}
    void* acquire(size_t bytes) override;
    void release(void* ptr, size_t bytes) override;
    void sync_device() override;
    void order_after(void* producer, void* consumer) override;
    int free_foreign(void* ptr, void* stream) override;
    uintptr_t place_canonical(uintptr_t lo, uintptr_t hi, size_t bytes, bool lines) override;

    // What was measured about the arenas handed to the pool (side_map.h).
    SideRegistry& sides() { return sides_; }
    // True when ptr is the start of an arena this backing store acquired and still holds.
    bool owns_arena(void* ptr) {
        std::lock_guard<std::mutex> lk(mu_);
        return raw_of_.count(ptr) != 0;
    }

private:
    int device_;
    SideRegistry sides_;
    std::mutex mu_;
    // aligned pointer handed to the pool -> pointer hipMalloc returned (they differ only when
    // the runtime did not return a 2 MiB-aligned address by itself)
    std::unordered_map<void*, void*> raw_of_;
};

}  // namespace sideaware
