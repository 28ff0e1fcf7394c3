#include "hip_backing.h"

#include <hip/hip_runtime_api.h>

#include <cstdio>

namespace sideaware {

namespace {
struct DeviceGuard {
    int prev = -1;
    bool switched = false;
    explicit DeviceGuard(int want) {
        if (hipGetDevice(&prev) == hipSuccess && prev != want) {
            switched = hipSetDevice(want) == hipSuccess;
        }
    }
    ~DeviceGuard() {
        if (switched) (void)hipSetDevice(prev);
    }
};
}  // namespace

// hipMalloc returns 2 MiB-aligned addresses for requests of this size on current ROCm, but
// nothing promises it, so a misaligned answer is replaced by an over-sized one whose aligned
// interior is handed out instead.
void* HipBacking::acquire(size_t bytes) {
    DeviceGuard g(device_);
    // The runtime may satisfy a request larger than the free device memory by spilling to host
    // memory; a device pool must answer "out of memory" instead.
    size_t free_bytes = 0, total_bytes = 0;
    if (hipMemGetInfo(&free_bytes, &total_bytes) == hipSuccess && bytes > free_bytes) return nullptr;
    void* raw = nullptr;
    if (hipMalloc(&raw, bytes) != hipSuccess) {
        (void)hipGetLastError();      // an out-of-memory answer must not poison later calls
        return nullptr;
    }
    void* aligned = raw;
    if ((uintptr_t)raw % kRegionAlign != 0) {
        (void)hipFree(raw);
        raw = nullptr;
        if (hipMalloc(&raw, bytes + kRegionAlign) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
        aligned = (void*)(((uintptr_t)raw + kRegionAlign - 1) / kRegionAlign * kRegionAlign);
    }
    {
        std::lock_guard<std::mutex> lk(mu_);
        raw_of_[aligned] = raw;
    }
    // which half of the device holds which granule of the new arena (a few timed loads)
    sides_.add_arena(aligned, bytes);
    return aligned;
}

void HipBacking::release(void* ptr, size_t) {
    sides_.remove_arena(ptr);
    void* raw = ptr;
    {
        std::lock_guard<std::mutex> lk(mu_);
        auto it = raw_of_.find(ptr);
        if (it != raw_of_.end()) {
            raw = it->second;
            raw_of_.erase(it);
        }
    }
    DeviceGuard g(device_);
    if (hipFree(raw) != hipSuccess) {
        std::fprintf(stderr, "sideaware: hipFree(%p) failed: %s\n", raw, hipGetErrorString(hipGetLastError()));
    }
}

// Where in the free run [lo, hi) a block of `bytes` should start so that its granules alternate
// between the device's halves the same way every other block's do; 0 when nothing is known about
// the arena the run lies in.
uintptr_t HipBacking::place_canonical(uintptr_t lo, uintptr_t hi, size_t bytes, bool lines) {
    uintptr_t base = 0;
    unsigned int flip = 0;
    if (!sides_.arena_of((const void*)lo, &base, &flip, /*placing=*/true)) return 0;
    return canonical_start(sides_.hash(), flip, base, lo, hi, bytes, lines);
}

void HipBacking::sync_device() {
    DeviceGuard g(device_);
    (void)hipDeviceSynchronize();
}

// The consumer stream waits, on the device, for what the producer stream has queued so far; the
// host does not block.  If the event cannot be made or recorded the host waits for the producer
// stream instead, and if even that is refused, for the whole device.
void HipBacking::order_after(void* producer, void* consumer) {
    DeviceGuard g(device_);
    hipEvent_t ev = nullptr;
    if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) == hipSuccess) {
        bool ordered = hipEventRecord(ev, (hipStream_t)producer) == hipSuccess &&
                       hipStreamWaitEvent((hipStream_t)consumer, ev, 0) == hipSuccess;
        (void)hipEventDestroy(ev);      // released by the runtime once the wait has been satisfied
        if (ordered) return;
    }
    (void)hipGetLastError();
    if (hipStreamSynchronize((hipStream_t)producer) != hipSuccess) {
        (void)hipGetLastError();
        (void)hipDeviceSynchronize();
    }
}

// A pointer the pool never handed out is released by the runtime behind the work already queued
// on `stream`, as the reference does with cudaFreeAsync (sideaware.cu:1258-1260).  Memory that did
// not come from the runtime's stream-ordered allocator may be refused there: then the stream is
// drained and the blocking free takes it.
int HipBacking::free_foreign(void* ptr, void* stream) {
    DeviceGuard g(device_);
    hipError_t e = hipFreeAsync(ptr, (hipStream_t)stream);
    if (e == hipSuccess) return 0;
    (void)hipGetLastError();
    (void)hipStreamSynchronize((hipStream_t)stream);
    e = hipFree(ptr);
    if (e != hipSuccess) (void)hipGetLastError();
    return (int)e;
}

}  // namespace sideaware
