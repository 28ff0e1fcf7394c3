#include "pool.h"

#include <algorithm>
#include <cassert>
#include <cstdio>

namespace sideaware {

namespace {
constexpr int kLinearClasses = 8;                 // 512 B .. 4 KiB in 512 B steps
constexpr int kStepsPerOctave = 8;                // above 4 KiB: 8 classes per power of two
constexpr int kFirstOctaveLog2 = 12;

inline int ceil_log2(size_t v) {                  // smallest k with 2^k >= v, v >= 1
    return v <= 1 ? 0 : 64 - __builtin_clzll((unsigned long long)(v - 1));
}
}  // namespace

size_t Pool::round_large(size_t bytes) {
    if (bytes == 0) bytes = 1;
    return (bytes + kRegionAlign - 1) / kRegionAlign * kRegionAlign;
}

// Small sizes round up to a class: multiples of 512 B up to 4 KiB, then eight evenly spaced
// classes per octave (at most 12.5 % internal slack), all multiples of 512 B.
size_t Pool::small_class_size(size_t bytes) {
    if (bytes <= kLinearClasses * kSmallGranule) {
        return bytes == 0 ? kSmallGranule : (bytes + kSmallGranule - 1) / kSmallGranule * kSmallGranule;
    }
    int k = ceil_log2(bytes);                      // bytes in (2^(k-1), 2^k]
    size_t step = (size_t)1 << (k - 1 - 3);
    return (bytes + step - 1) / step * step;
}

int Pool::small_class_index(size_t bytes) {
    size_t c = small_class_size(bytes);
    if (c <= kLinearClasses * kSmallGranule) return (int)(c / kSmallGranule) - 1;
    int k = ceil_log2(c);                          // c in (2^(k-1), 2^k]
    size_t step = (size_t)1 << (k - 1 - 3);
    int sub = (int)(c / step) - kStepsPerOctave;   // 1..8
    return kLinearClasses + (k - 1 - kFirstOctaveLog2) * kStepsPerOctave + (sub - 1);
}

Pool::Pool(Backing* backing) : backing_(backing) {
    small_.resize(kLinearClasses + (64 - kFirstOctaveLog2) * kStepsPerOctave);
}

Pool::~Pool() {
    // Device memory is left to process teardown: the runtime may already be gone when static
    // destructors run, and freeing through it then is worse than not freeing.
}

void Pool::set_large_threshold(size_t bytes) {
    std::lock_guard<std::mutex> g(mu_);
    large_threshold_ = bytes;
}

void Pool::set_trim_thresholds(size_t start_bytes, size_t end_bytes) {
    std::lock_guard<std::mutex> g(mu_);
    trim_start_ = start_bytes;
    trim_end_ = std::min(end_bytes, start_bytes);
}

void Pool::set_reserve_limit(size_t bytes) {
    std::lock_guard<std::mutex> g(mu_);
    reserve_limit_ = bytes;
}

void* Pool::backing_acquire_locked(size_t bytes) {
    st_.backing_acquires++;
    if (reserve_limit_ && st_.bytes_reserved + bytes > reserve_limit_) return nullptr;
    return backing_->acquire(bytes);
}

void Pool::note_reserved(int64_t delta) {
    st_.bytes_reserved = (uint64_t)((int64_t)st_.bytes_reserved + delta);
    st_.peak_reserved = std::max(st_.peak_reserved, st_.bytes_reserved);
}

// ---------------------------------------------------------------------------------------------
// Large path
// ---------------------------------------------------------------------------------------------

// Hands cached large blocks back to the backing store until at most `down_to` bytes remain
// cached.  Mirrors unmap_free_allocations (sideaware.cu:873-906): the device is drained first,
// because a cached block may still be in use by work queued before it was freed.
size_t Pool::trim_large_locked(size_t down_to) {
    if (st_.bytes_cached_large <= down_to) return 0;
    backing_->sync_device();
    st_.device_syncs++;
    size_t released = 0;
    for (auto it = large_cache_.begin(); it != large_cache_.end() && st_.bytes_cached_large > down_to;) {
        auto& vec = it->second;
        // oldest first: the most recently freed blocks are the likeliest to be asked for again
        size_t n = 0;
        while (n < vec.size() && st_.bytes_cached_large > down_to) {
            backing_->release(vec[n].ptr, vec[n].bytes);
            st_.backing_releases++;
            st_.bytes_cached_large -= vec[n].bytes;
            note_reserved(-(int64_t)vec[n].bytes);
            released += vec[n].bytes;
            n++;
        }
        vec.erase(vec.begin(), vec.begin() + n);
        if (vec.empty()) it = large_cache_.erase(it); else ++it;
    }
    return released;
}

void* Pool::acquire_large_locked(size_t rounded, void* stream) {
    void* p = backing_acquire_locked(rounded);
    if (!p) return nullptr;
    assert(((uintptr_t)p % kRegionAlign) == 0);
    note_reserved((int64_t)rounded);
    LargeBlock blk;
    blk.ptr = p;
    blk.bytes = rounded;
    blk.last_stream = stream;
    large_live_.emplace(p, blk);
    st_.bytes_live += rounded;
    return p;
}

void* Pool::allocate_large_locked(size_t bytes, void* stream) {
    const size_t rounded = round_large(bytes);

    // 1) exact-size reuse, newest first (sideaware.cu:1199-1219); failing that, the smallest
    //    cached region that is at most one eighth larger, handed out whole.  Any 2 MiB-aligned
    //    region serves, and a driver allocation costs hundreds of microseconds.
    auto it = large_cache_.lower_bound(rounded);
    while (it != large_cache_.end() && it->second.empty()) ++it;
    if (it != large_cache_.end() && it->first <= rounded + rounded / 8) {
        LargeBlock blk = it->second.back();
        it->second.pop_back();
        if (it->second.empty()) large_cache_.erase(it);
        st_.bytes_cached_large -= blk.bytes;
        if (blk.last_stream != stream) {
            backing_->sync_stream(blk.last_stream);
            st_.stream_syncs++;
            blk.last_stream = stream;
        }
        large_live_.emplace(blk.ptr, blk);
        st_.bytes_live += blk.bytes;
        st_.large_hits++;
        return blk.ptr;
    }
    st_.large_misses++;

    // 2) trim the cache if it has outgrown its budget, then ask the backing store
    if (st_.bytes_cached_large > trim_start_) {
        trim_large_locked(trim_end_);
        st_.trims++;
    }
    if (void* p = acquire_large_locked(rounded, stream)) return p;

    // 3) give back every cached large block and retry
    st_.ladder_retries++;
    trim_large_locked(0);
    if (void* p = acquire_large_locked(rounded, stream)) return p;

    // 4) give back empty slabs too and retry one last time
    st_.ladder_retries++;
    release_empty_slabs_locked();
    if (void* p = acquire_large_locked(rounded, stream)) return p;

    st_.failures++;
    return nullptr;
}

// ---------------------------------------------------------------------------------------------
// Small path
// ---------------------------------------------------------------------------------------------

Pool::Slab* Pool::new_slab_locked(size_t block) {
    size_t want = std::min(std::max(block * 16, kRegionAlign), kMaxSlabBytes);
    want = std::max(want, block);
    size_t bytes = round_large(want);
    void* p = backing_acquire_locked(bytes);
    if (!p) {
        // the same ladder as the large path, compressed: drop caches, then retry once
        st_.ladder_retries++;
        trim_large_locked(0);
        release_empty_slabs_locked();
        p = backing_acquire_locked(bytes);
        if (!p) return nullptr;
    }
    note_reserved((int64_t)bytes);
    st_.slabs_acquired++;
    auto slab = std::make_unique<Slab>();
    slab->base = (char*)p;
    slab->bytes = bytes;
    slab->block = block;
    slab->capacity = (uint32_t)(bytes / block);
    slab->in_use.assign(slab->capacity, 0);
    for (size_t off = 0; off < bytes; off += kRegionAlign) {
        slab_by_page_[((uintptr_t)p + off) / kRegionAlign] = slab.get();
    }
    st_.bytes_cached_small += (uint64_t)slab->capacity * block;
    Slab* raw = slab.get();
    slab_store_.push_back(std::move(slab));
    return raw;
}

void* Pool::allocate_small_locked(size_t bytes, void* stream) {
    const size_t block = small_class_size(bytes);
    SmallClass& cls = small_[small_class_index(bytes)];

    void* p = nullptr;
    if (!cls.free.empty()) {
        FreeSmall f = cls.free.back();
        cls.free.pop_back();
        if (f.stream != stream) {
            backing_->sync_stream(f.stream);
            st_.stream_syncs++;
        }
        p = f.ptr;
        st_.small_hits++;
    } else {
        if (!cls.bump || cls.bump->carved == cls.bump->capacity) {
            cls.bump = new_slab_locked(block);
            if (!cls.bump) {
                st_.failures++;
                return nullptr;
            }
            cls.slabs.push_back(cls.bump);
        }
        p = cls.bump->base + (size_t)cls.bump->carved * block;
        cls.bump->carved++;
        st_.small_carves++;
    }
    Slab* slab = slab_by_page_[(uintptr_t)p / kRegionAlign];
    size_t idx = ((char*)p - slab->base) / block;
    assert(!slab->in_use[idx]);
    slab->in_use[idx] = 1;
    slab->live++;
    st_.bytes_live += block;
    st_.bytes_cached_small -= block;
    return p;
}

// Gives back every slab with no live block.  Their blocks are purged from the class free lists
// first; a slab that is only partly used stays.
size_t Pool::release_empty_slabs_locked() {
    bool any = false;
    for (auto& s : slab_store_) any |= (s->live == 0);
    if (!any) return 0;
    backing_->sync_device();
    st_.device_syncs++;
    size_t released = 0;
    for (auto& cls : small_) {
        if (cls.slabs.empty()) continue;
        auto dead = [&](void* ptr) {
            Slab* s = slab_by_page_[(uintptr_t)ptr / kRegionAlign];
            return s->live == 0;
        };
        cls.free.erase(std::remove_if(cls.free.begin(), cls.free.end(),
                                      [&](const FreeSmall& f) { return dead(f.ptr); }),
                       cls.free.end());
        if (cls.bump && cls.bump->live == 0) cls.bump = nullptr;
        cls.slabs.erase(std::remove_if(cls.slabs.begin(), cls.slabs.end(),
                                       [](Slab* s) { return s->live == 0; }),
                        cls.slabs.end());
        // an older slab with an untouched tail can serve as the bump slab again
        if (!cls.bump) {
            for (Slab* s : cls.slabs) if (s->carved < s->capacity) { cls.bump = s; break; }
        }
    }
    for (auto it = slab_store_.begin(); it != slab_store_.end();) {
        Slab* s = it->get();
        if (s->live != 0) { ++it; continue; }
        for (size_t off = 0; off < s->bytes; off += kRegionAlign) {
            slab_by_page_.erase(((uintptr_t)s->base + off) / kRegionAlign);
        }
        backing_->release(s->base, s->bytes);
        st_.backing_releases++;
        st_.bytes_cached_small -= (uint64_t)s->capacity * s->block;
        note_reserved(-(int64_t)s->bytes);
        released += s->bytes;
        it = slab_store_.erase(it);
    }
    return released;
}

// ---------------------------------------------------------------------------------------------
// Public entry points
// ---------------------------------------------------------------------------------------------

void* Pool::allocate(size_t bytes, void* stream, bool always_large) {
    std::lock_guard<std::mutex> g(mu_);
    if (always_large || bytes >= large_threshold_) return allocate_large_locked(bytes, stream);
    return allocate_small_locked(bytes, stream);
}

int Pool::deallocate(void* ptr, void* stream) {
    if (!ptr) return 0;
    std::unique_lock<std::mutex> g(mu_);

    auto it = large_live_.find(ptr);
    if (it != large_live_.end()) {
        LargeBlock blk = it->second;
        large_live_.erase(it);
        blk.last_stream = stream;
        st_.bytes_live -= blk.bytes;
        st_.bytes_cached_large += blk.bytes;
        large_cache_[blk.bytes].push_back(blk);
        return 0;
    }

    auto sit = slab_by_page_.find((uintptr_t)ptr / kRegionAlign);
    if (sit != slab_by_page_.end()) {
        Slab* slab = sit->second;
        size_t off = (char*)ptr - slab->base;
        size_t idx = off / slab->block;
        if (off % slab->block != 0 || idx >= slab->carved || !slab->in_use[idx]) {
            std::fprintf(stderr, "sideaware: free of %p, which is not a live block of this pool\n", ptr);
            return 1;
        }
        slab->in_use[idx] = 0;
        slab->live--;
        st_.bytes_live -= slab->block;
        st_.bytes_cached_small += slab->block;
        small_[small_class_index(slab->block)].free.push_back({ptr, stream});
        return 0;
    }

    // Not ours (sideaware.cu:1258-1260 forwards unknown pointers to cudaFreeAsync).
    st_.foreign_frees++;
    g.unlock();
    return backing_->free_foreign(ptr, stream);
}

size_t Pool::release_unused() {
    std::lock_guard<std::mutex> g(mu_);
    size_t n = trim_large_locked(0);
    n += release_empty_slabs_locked();
    return n;
}

PoolStats Pool::stats() {
    std::lock_guard<std::mutex> g(mu_);
    return st_;
}

size_t Pool::block_bytes(void* ptr) {
    std::lock_guard<std::mutex> g(mu_);
    auto it = large_live_.find(ptr);
    if (it != large_live_.end()) return it->second.bytes;
    auto sit = slab_by_page_.find((uintptr_t)ptr / kRegionAlign);
    if (sit == slab_by_page_.end()) return 0;
    Slab* slab = sit->second;
    size_t off = (char*)ptr - slab->base;
    bool live = off % slab->block == 0 && off / slab->block < slab->carved && slab->in_use[off / slab->block];
    return live ? slab->block : 0;
}

bool Pool::owns_live(void* ptr) {
    std::lock_guard<std::mutex> g(mu_);
    if (large_live_.count(ptr)) return true;
    auto sit = slab_by_page_.find((uintptr_t)ptr / kRegionAlign);
    if (sit == slab_by_page_.end()) return false;
    Slab* slab = sit->second;
    size_t off = (char*)ptr - slab->base;
    return off % slab->block == 0 && off / slab->block < slab->carved && slab->in_use[off / slab->block];
}

}  // namespace sideaware
