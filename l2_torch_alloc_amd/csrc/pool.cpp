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

void Pool::set_arena_bytes(size_t bytes) {
    std::lock_guard<std::mutex> g(mu_);
    arena_bytes_ = bytes ? round_large(bytes) : 0;
}

void Pool::note_reserved(int64_t delta) {
    st_.bytes_reserved = (uint64_t)((int64_t)st_.bytes_reserved + delta);
    st_.peak_reserved = std::max(st_.peak_reserved, st_.bytes_reserved);
}

// ---------------------------------------------------------------------------------------------
// Large path
// ---------------------------------------------------------------------------------------------

// Adds a free extent, merging it with free neighbours of the same arena.
void Pool::extent_insert_locked(int kind, uintptr_t addr, Extent e) {
    ExtentIndex& ix = free_[kind];
    auto erase_size = [&](size_t bytes, uintptr_t a) { ix.by_size.erase({bytes, a}); };
    auto next = ix.by_addr.lower_bound(addr);
    if (next != ix.by_addr.end() && next->second.arena == e.arena && addr + e.bytes == next->first) {
        e.freed_on.merge(next->second.freed_on);
        e.bytes += next->second.bytes;
        erase_size(next->second.bytes, next->first);
        next = ix.by_addr.erase(next);
    }
    if (next != ix.by_addr.begin()) {
        auto prev = std::prev(next);
        if (prev->second.arena == e.arena && prev->first + prev->second.bytes == addr) {
            e.freed_on.merge(prev->second.freed_on);
            addr = prev->first;
            e.bytes += prev->second.bytes;
            erase_size(prev->second.bytes, prev->first);
            ix.by_addr.erase(prev);
        }
    }
    ix.by_addr[addr] = e;
    ix.by_size.emplace(e.bytes, addr);
}

// Takes `bytes` from the best-fitting free extent; what is left of it stays free.  Normally the
// block is the extent's front.  With `canonical` the backing store is asked where in the extent the
// block should start so that the device's memory halves alternate through it like through every
// other block placed this way (Backing::place_canonical); the first few extents in best-fit order
// are tried, and when none can hold such a block without a large hole in front of it (or the
// backing store knows no rule) the front of the best fit is taken after all.
bool Pool::extent_take_locked(int kind, size_t bytes, uintptr_t* addr, Extent* taken, bool canonical) {
    ExtentIndex& ix = free_[kind];
    auto sit = ix.by_size.lower_bound({bytes, 0});
    if (sit == ix.by_size.end()) return false;
    uintptr_t start = sit->second;
    if (canonical) {
        bool placed = false;
        int tries = 0;
        for (auto cand = sit; cand != ix.by_size.end() && tries < kCanonicalTries; ++cand, ++tries) {
            const uintptr_t at = backing_->place_canonical(cand->second, cand->second + cand->first, bytes, /*lines=*/true);
            if (at == 0) continue;
            assert(at >= cand->second && at + bytes <= cand->second + cand->first && at % kRegionAlign == 0);
            const size_t divisor = bytes <= kCanonicalSmallBytes ? kCanonicalGapDivisorSmall
                                 : bytes <= 2 * kCanonicalSmallBytes ? kCanonicalGapDivisorMid : kCanonicalGapDivisor;
            if (at - cand->second > std::max<size_t>(kCanonicalSlack, bytes / divisor)) continue;   // too large a hole in front
            sit = cand;
            start = at;
            placed = true;
            break;
        }
        if (!placed) {
            // the best fit after all, but at least on the right starting page: the block then follows
            // the pattern up to the first 256 MiB line it meets
            const uintptr_t at = backing_->place_canonical(sit->second, sit->second + sit->first, bytes, /*lines=*/false);
            if (at != 0) {
                assert(at >= sit->second && at + bytes <= sit->second + sit->first && at % kRegionAlign == 0);
                start = at;
            }
        }
        if (placed) st_.canonical_placements++;
    }
    const uintptr_t ext_addr = sit->second;
    auto ait = ix.by_addr.find(ext_addr);
    *taken = ait->second;
    *addr = start;
    ix.by_size.erase(sit);
    ix.by_addr.erase(ait);
    if (start > ext_addr) {
        Extent front = *taken;
        front.bytes = start - ext_addr;
        ix.by_addr[ext_addr] = front;
        ix.by_size.emplace(front.bytes, ext_addr);
    }
    if (ext_addr + taken->bytes > start + bytes) {
        Extent rest = *taken;
        rest.bytes = ext_addr + taken->bytes - (start + bytes);
        ix.by_addr[start + bytes] = rest;
        ix.by_size.emplace(rest.bytes, start + bytes);
    }
    (kind == kSlabArenas ? st_.bytes_free_slab_arena : st_.bytes_free_arena) -= bytes;
    return true;
}

// Best fit from the free extents of the large regions' arenas.  The taking stream is ordered
// after every other stream the extent's pages were freed on (stream order, as for a cached
// region).
void* Pool::carve_locked(size_t rounded, void* stream) {
    uintptr_t addr;
    Extent e;
    if (!extent_take_locked(kLargeArenas, rounded, &addr, &e, rounded >= kCanonicalMinBytes)) return nullptr;
    if (e.freed_on.overflow) {
        backing_->sync_device();
        st_.device_syncs++;
    } else {
        for (int i = 0; i < e.freed_on.count; i++) {
            if (e.freed_on.streams[i] == stream) continue;
            backing_->order_after(e.freed_on.streams[i], stream);
            st_.stream_syncs++;
        }
    }
    LargeBlock blk;
    blk.ptr = (void*)addr;
    blk.bytes = rounded;
    blk.last_stream = stream;
    blk.arena = e.arena;
    large_live_.emplace(blk.ptr, blk);
    st_.bytes_live += rounded;
    return blk.ptr;
}

// A fresh arena from the backing store: the configured size (for slabs at most
// kMaxSlabArenaBytes), or just the request if that is larger, or if the backing store cannot
// give the configured size any more.
bool Pool::new_arena_locked(int kind, size_t min_bytes) {
    size_t configured = kind == kSlabArenas ? std::min(arena_bytes_, kMaxSlabArenaBytes) : arena_bytes_;
    // a region that gets an arena of its own still needs room to start on the right page parity
    size_t padded = min_bytes;
    if (kind == kLargeArenas && arena_bytes_ != 0 && min_bytes >= kCanonicalMinBytes && min_bytes + kCanonicalSlack > configured) {
        padded = min_bytes + kCanonicalSlack;
    }
    size_t want = std::max(configured, padded);
    void* p = backing_acquire_locked(want);
    if (!p && want > padded) {
        want = padded;
        p = backing_acquire_locked(want);
    }
    if (!p && padded > min_bytes) {
        want = min_bytes;
        p = backing_acquire_locked(want);
    }
    if (!p) return false;
    assert(((uintptr_t)p % kRegionAlign) == 0);
    note_reserved((int64_t)want);
    st_.arenas_acquired++;
    auto arena = std::make_unique<Arena>();
    arena->base = (char*)p;
    arena->bytes = want;
    arena->for_slabs = kind == kSlabArenas;
    Extent e;
    e.bytes = want;
    e.arena = arena.get();
    // e.freed_on stays empty: never used, nothing to wait for
    (kind == kSlabArenas ? st_.bytes_free_slab_arena : st_.bytes_free_arena) += want;
    extent_insert_locked(kind, (uintptr_t)p, e);
    arenas_.push_back(std::move(arena));
    return true;
}

// Folds every cached region back into its arena's free extents.
void Pool::flush_cache_locked() {
    for (auto& kv : large_cache_) {
        for (LargeBlock& blk : kv.second) {
            Extent e;
            e.bytes = blk.bytes;
            e.arena = blk.arena;
            e.freed_on.add(blk.last_stream);
            st_.bytes_free_arena += blk.bytes;
            extent_insert_locked(kLargeArenas, (uintptr_t)blk.ptr, e);
        }
    }
    large_cache_.clear();
    st_.bytes_cached_large = 0;
}

// Returns wholly free arenas of one kind to the backing store until at most `down_to` free bytes
// remain in that kind's arenas.  The device is drained first (unmap_free_allocations does the
// same, sideaware.cu:873-906): freed pages may still be in use by work queued before the free.
size_t Pool::release_free_arenas_locked(int kind, size_t down_to, bool device_idle) {
    ExtentIndex& ix = free_[kind];
    uint64_t& free_bytes = kind == kSlabArenas ? st_.bytes_free_slab_arena : st_.bytes_free_arena;
    size_t released = 0;
    bool synced = device_idle;
    for (auto it = arenas_.begin(); it != arenas_.end() && free_bytes > down_to;) {
        Arena* a = it->get();
        if (a->for_slabs != (kind == kSlabArenas)) { ++it; continue; }
        auto fit = ix.by_addr.find((uintptr_t)a->base);
        if (fit == ix.by_addr.end() || fit->second.bytes != a->bytes) { ++it; continue; }
        if (!synced) {
            backing_->sync_device();
            st_.device_syncs++;
            synced = true;
        }
        ix.by_size.erase({a->bytes, (uintptr_t)a->base});
        ix.by_addr.erase(fit);
        backing_->release(a->base, a->bytes);
        st_.backing_releases++;
        free_bytes -= a->bytes;
        note_reserved(-(int64_t)a->bytes);
        released += a->bytes;
        it = arenas_.erase(it);
    }
    return released;
}

// Brings cached + free large bytes down to `down_to` (as far as whole arenas allow).
size_t Pool::trim_large_locked(size_t down_to) {
    if (st_.bytes_cached_large + st_.bytes_free_arena <= down_to) return 0;
    flush_cache_locked();
    return release_free_arenas_locked(kLargeArenas, down_to);
}

void* Pool::allocate_large_locked(size_t bytes, void* stream) {
    const size_t rounded = round_large(bytes);

    bool trimmed = false;
    // 1) exact-size reuse, newest first (sideaware.cu:1199-1219)
    auto it = large_cache_.find(rounded);
    if (it == large_cache_.end() || it->second.empty()) {
        if (arena_bytes_ != 0) {
            // 2) with arenas: every cached region goes back into its arena's free extents, where
            //    neighbours merge, and the request is carved, best fit, from what is free then.  No
            //    waste, no driver call; a fold costs microseconds.  Folding before every carve (and
            //    not only when nothing else fits) is what keeps the arenas whole: a cached region
            //    is a hole its neighbours cannot merge across, and carving around such holes left
            //    16 GB of a 89 GB pool free yet too fragmented for a 512 MiB request in a churn of
            //    10,000 requests; folding first, the same churn peaks at 76 GB.
            //    When cached + free bytes have outgrown their budget the same moment is the
            //    reference's threshold trim (sideaware.cu:1242): wholly free arenas go home too.
            if (st_.bytes_cached_large + st_.bytes_free_arena > trim_start_) {
                trim_large_locked(trim_end_);
                st_.trims++;
                trimmed = true;
            } else if (!large_cache_.empty()) {
                flush_cache_locked();
                st_.cache_folds++;
            }
            if (void* p = carve_locked(rounded, stream)) {
                st_.large_carves++;
                return p;
            }
            it = large_cache_.end();
        } else {
            // 2') without arenas every region is a backing allocation of its own: the smallest
            //     cached region at most one eighth larger is handed out whole
            it = large_cache_.lower_bound(rounded);
            while (it != large_cache_.end() && it->second.empty()) ++it;
            if (it != large_cache_.end() && it->first > rounded + rounded / 8) it = large_cache_.end();
        }
    }
    if (it != large_cache_.end() && !it->second.empty()) {
        LargeBlock blk = it->second.back();
        it->second.pop_back();
        if (it->second.empty()) large_cache_.erase(it);
        st_.bytes_cached_large -= blk.bytes;
        if (blk.last_stream != stream) {
            backing_->order_after(blk.last_stream, stream);
            st_.stream_syncs++;
            blk.last_stream = stream;
        }
        large_live_.emplace(blk.ptr, blk);
        st_.bytes_live += blk.bytes;
        st_.large_hits++;
        return blk.ptr;
    }
    st_.large_misses++;

    // 4) a miss.  If cached + free bytes have outgrown their budget, fold the cache into the
    //    arenas and give wholly free arenas back (the reference's threshold trim,
    //    sideaware.cu:1242); what stays free may now fit the request.
    if (!trimmed && st_.bytes_cached_large + st_.bytes_free_arena > trim_start_) {
        trim_large_locked(trim_end_);
        st_.trims++;
        if (void* p = carve_locked(rounded, stream)) return p;
    }
    if (new_arena_locked(kLargeArenas, rounded)) return carve_locked(rounded, stream);

    // 5) the backing store refused: fold the cache back, carve if that made room, else give every
    //    free arena back and retry
    st_.ladder_retries++;
    flush_cache_locked();
    if (void* p = carve_locked(rounded, stream)) return p;
    release_free_arenas_locked(kLargeArenas, 0);
    if (new_arena_locked(kLargeArenas, rounded)) return carve_locked(rounded, stream);

    // 6) give back empty slabs too and retry one last time
    st_.ladder_retries++;
    release_empty_slabs_locked();
    if (new_arena_locked(kLargeArenas, rounded)) return carve_locked(rounded, stream);

    st_.failures++;
    return nullptr;
}

// ---------------------------------------------------------------------------------------------
// Small path
// ---------------------------------------------------------------------------------------------

// Memory for one slab: carved from the slabs' arenas (a new one when none has room), or a
// backing allocation of its own when arenas are switched off.  Extents in the slabs' arenas are
// only ever freed after a device sync, so a carve there never has a stream to wait for.
void* Pool::slab_memory_locked(size_t bytes, Arena** arena) {
    *arena = nullptr;
    if (arena_bytes_ == 0) {
        void* p = backing_acquire_locked(bytes);
        if (p) note_reserved((int64_t)bytes);
        return p;
    }
    uintptr_t addr;
    Extent e;
    if (!extent_take_locked(kSlabArenas, bytes, &addr, &e, false)) {
        if (!new_arena_locked(kSlabArenas, bytes)) return nullptr;
        if (!extent_take_locked(kSlabArenas, bytes, &addr, &e, false)) return nullptr;
    }
    *arena = e.arena;
    return (void*)addr;
}

Pool::Slab* Pool::new_slab_locked(size_t block) {
    size_t want = std::min(std::max(block * 16, kRegionAlign), kMaxSlabBytes);
    want = std::max(want, block);
    size_t bytes = round_large(want);
    Arena* arena = nullptr;
    void* p = slab_memory_locked(bytes, &arena);
    if (!p) {
        // the same ladder as the large path, compressed: drop caches, then retry once
        st_.ladder_retries++;
        trim_large_locked(0);
        release_empty_slabs_locked();
        p = slab_memory_locked(bytes, &arena);
        if (!p && round_large(block) < bytes) {
            bytes = round_large(block);      // last resort: a slab of a single block
            p = slab_memory_locked(bytes, &arena);
        }
        if (!p) return nullptr;
    }
    st_.slabs_acquired++;
    auto slab = std::make_unique<Slab>();
    slab->base = (char*)p;
    slab->bytes = bytes;
    slab->block = block;
    slab->arena = arena;
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
            backing_->order_after(f.stream, stream);
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

// Gives back every slab with no live block, and then every arena of slabs that is wholly free;
// returns the bytes that went back to the backing store.  The slabs' blocks are purged from the
// class free lists first; a slab that is only partly used stays.
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
        st_.bytes_cached_small -= (uint64_t)s->capacity * s->block;
        if (s->arena) {
            Extent e;
            e.bytes = s->bytes;
            e.arena = s->arena;
            // e.freed_on stays empty: the device was drained above
            st_.bytes_free_slab_arena += s->bytes;
            extent_insert_locked(kSlabArenas, (uintptr_t)s->base, e);
        } else {
            backing_->release(s->base, s->bytes);
            st_.backing_releases++;
            note_reserved(-(int64_t)s->bytes);
            released += s->bytes;
        }
        it = slab_store_.erase(it);
    }
    released += release_free_arenas_locked(kSlabArenas, 0, /*device_idle=*/true);
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
            st_.refused_frees++;
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

    // An address inside one of the pool's own arenas that is not a live block: a second free of a
    // large region, an interior pointer, a pointer into free pages.  The runtime must never see
    // it: an arena's first region starts at the arena's base, and the runtime's free of that
    // address would take the whole arena away from under every block carved from it.
    for (const auto& a : arenas_) {
        if ((char*)ptr >= a->base && (char*)ptr < a->base + a->bytes) {
            st_.refused_frees++;
            std::fprintf(stderr, "sideaware: free of %p, which is not a live block of this pool\n", ptr);
            return 1;
        }
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
