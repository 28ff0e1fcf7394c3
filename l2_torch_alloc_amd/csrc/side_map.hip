#include "side_map.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>

namespace sideaware {

// ---------------------------------------------------------------------------------------------
// Measurement
// ---------------------------------------------------------------------------------------------

namespace {

constexpr int kProbeLoads = 4;              // timed loads per sample; the first also pays for the address translation
constexpr size_t kScrubBytes = 128ull << 20;   // read after the first pass: four times the XCDs' L2s together
constexpr int kProbeGroups = 8;             // one workgroup per XCD, whatever the dealing offset

// Lane 0 of each workgroup times single loads, one at a time, inside the granule at base +
// offsets[i]: every XCD and every repeat has a 128-byte line of its own (line 8 * repeat + XCD of the
// granule's 64), so no load is answered by a line another one brought in, and the XCDs walk the
// samples in different rotations, so they do not queue up behind each other at one memory channel.
// The fastest repeat after the first (which also pays for the address translation) is kept.
// lat is [16][n], indexed by the XCD the workgroup found itself on.
__global__ __launch_bounds__(64) void sa_side_probe(const char* base, const uint64_t* offsets, int n, unsigned int* lat) {
    unsigned int xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    xcc &= 0xfu;
    if (threadIdx.x != 0) return;
    int acc = 0;
    const int start = (int)(((unsigned long long)(xcc & 7u) * (unsigned)n) / 8u);
    for (int step = 0; step < n; step++) {
        const int i = (start + step) % n;
        unsigned int best = ~0u;
        for (int k = 0; k < kProbeLoads; k++) {
            const int* ptr = (const int*)(base + offsets[i] + (size_t)(k * 8 + (int)(xcc & 7u)) * 128);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            unsigned long long t0 = __builtin_amdgcn_s_memtime();
            asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(t0) :: "memory");
            int v;
            asm volatile("global_load_dword %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(ptr) : "memory");
            unsigned long long t1 = __builtin_amdgcn_s_memtime();
            asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(t1) :: "memory");
            acc ^= v;
            const unsigned int d = (unsigned int)(t1 - t0);
            if (k > 0 && d < best) best = d;
        }
        lat[(size_t)xcc * n + i] = best;
    }
    if (acc == 0x12345678) lat[0] = (unsigned int)acc;      // keeps the loads alive
}

// Reads `vectors` 16-byte vectors once: pushes whatever the XCDs' L2s held out of them.
typedef int sa_probe_v4i __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void sa_side_scrub(const sa_probe_v4i* p, size_t vectors, unsigned int* sink) {
    sa_probe_v4i acc = {0, 0, 0, 0};
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < vectors; i += (size_t)gridDim.x * 256) acc ^= p[i];
    if ((acc.x ^ acc.y) == 0x5a5a5a5a && (acc.z ^ acc.w) == 0x5a5a5a5a && acc.x == acc.z) sink[0] = 1;
}

// The sample granules of the probe entry points: sample i of a region of `granules` granules is
// granule splitmix64(seed + i) % granules, so that host and device agree on them without a table.
__host__ __device__ inline unsigned long long sa_sample_granule(unsigned long long seed, unsigned int i,
                                                                unsigned long long granules) {
    unsigned long long z = (seed + (unsigned long long)i) * 0x9e3779b97f4a7c15ull + 0x9e3779b97f4a7c15ull;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    z ^= z >> 31;
    return z % granules;
}

// sa_side_probe with the sample offsets computed on the device (no table to upload).
__global__ __launch_bounds__(64) void sa_side_probe_seeded(const char* base, unsigned long long granules,
                                                           unsigned long long seed, int n, unsigned int* lat) {
    unsigned int xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    xcc &= 0xfu;
    if (threadIdx.x != 0) return;
    int acc = 0;
    const int start = (int)(((unsigned long long)(xcc & 7u) * (unsigned)n) / 8u);
    for (int step = 0; step < n; step++) {
        const int i = (start + step) % n;
        const unsigned long long offset = sa_sample_granule(seed, (unsigned int)i, granules) << kSideGranuleLog2;
        unsigned int best = ~0u;
        for (int k = 0; k < kProbeLoads; k++) {
            const int* ptr = (const int*)(base + offset + (size_t)(k * 8 + (int)(xcc & 7u)) * 128);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            unsigned long long t0 = __builtin_amdgcn_s_memtime();
            asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(t0) :: "memory");
            int v;
            asm volatile("global_load_dword %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(ptr) : "memory");
            unsigned long long t1 = __builtin_amdgcn_s_memtime();
            asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(t1) :: "memory");
            acc ^= v;
            const unsigned int d = (unsigned int)(t1 - t0);
            if (k > 0 && d < best) best = d;
        }
        lat[(size_t)xcc * n + i] = best;
    }
    if (acc == 0x12345678) lat[0] = (unsigned int)acc;
}

// Clears the probe's scratch with a kernel (a memset node recorded into a captured graph is the
// one thing the graphs of this platform replay wrongly).
__global__ __launch_bounds__(256) void sa_side_clear(unsigned int* p, int words) {
    const int i = (int)(blockIdx.x * 256 + threadIdx.x);
    if (i < words) p[i] = 0;
}

// One thread per sample: the middle of each half's times, and which half is clearly faster.
__global__ __launch_bounds__(64) void sa_side_classify(const unsigned int* lat, int n, int* sides) {
    const int i = (int)(blockIdx.x * 64 + threadIdx.x);
    if (i >= n) return;
    float mid[2];
    bool ok = true;
    for (int h = 0; h < 2; h++) {
        unsigned int v[4];
        int cnt = 0;
        for (int x = 0; x < 4; x++) {
            const unsigned int t = lat[(size_t)(h * 4 + x) * n + i];
            if (t != 0 && t != ~0u) v[cnt++] = t;
        }
        if (cnt < 3) { ok = false; break; }
        for (int a = 1; a < cnt; a++) for (int b = a; b > 0 && v[b] < v[b - 1]; b--) { unsigned int t = v[b]; v[b] = v[b - 1]; v[b - 1] = t; }
        mid[h] = cnt == 4 ? 0.5f * ((float)v[1] + (float)v[2]) : (float)v[1];
    }
    int side = -1;
    if (ok) {
        const float lo = mid[0] < mid[1] ? mid[0] : mid[1], hi = mid[0] < mid[1] ? mid[1] : mid[0];
        if (hi - lo >= 0.2f * lo) side = mid[0] < mid[1] ? 0 : 1;      // near about 450 cycles, far about 680
    }
    sides[i] = side;
}

struct DeviceGuard {
    int prev = -1;
    bool switched = false;
    explicit DeviceGuard(int want) {
        if (hipGetDevice(&prev) == hipSuccess && prev != want) switched = hipSetDevice(want) == hipSuccess;
    }
    ~DeviceGuard() { if (switched) (void)hipSetDevice(prev); }
};

// A thread that is capturing a stream in the global mode may not launch on another stream: the
// probe switches the thread to the relaxed mode for its own launches.
struct RelaxedCapture {
    hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
    bool exchanged = false;
    RelaxedCapture() { exchanged = hipThreadExchangeStreamCaptureMode(&mode) == hipSuccess; if (!exchanged) (void)hipGetLastError(); }
    ~RelaxedCapture() { if (exchanged) (void)hipThreadExchangeStreamCaptureMode(&mode); }
};

bool side_debug() {
    static const bool on = [] { const char* v = std::getenv("SIDEAWARE_SIDE_DEBUG"); return v && v[0] == '1'; }();
    return on;
}

bool side_probing_enabled() {
    const char* v = std::getenv("SIDEAWARE_SIDE_PROBE");
    return !(v && v[0] == '0');
}

}  // namespace

// The allocation-free probe's scratch: the per-XCD times of up to kNoAllocMaxSamples samples plus
// the scrub kernel's sink.  One copy per device the library runs on, held until the process ends.
static __device__ __align__(256) unsigned int scratch[16 * SideRegistry::kNoAllocMaxSamples + 64];

void SideRegistry::init_static_scratch() {
    std::lock_guard<std::mutex> g(mu_);
    if (static_scratch_) return;
    DeviceGuard dev(device_);
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess) {
        (void)hipGetLastError();
        return;
    }
    static_scratch_ = (unsigned int*)ptr;            // this device's copy of the array
}

// The words captured launches read their dealing offset from, and the kernel that writes one: a
// single wave, captured ahead of the launches that read the word, on the same stream.
static __device__ __align__(256) unsigned int capture_words[SideRegistry::kCaptureWords];

__global__ __launch_bounds__(64) void sa_scout(unsigned int* word) {
    unsigned int xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    if (threadIdx.x == 0) *word = 0x80000000u | (xcc & 0xfu);
}

void SideRegistry::init_capture_words() {
    std::lock_guard<std::mutex> g(mu_);
    if (capture_words_) return;
    DeviceGuard dev(device_);
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(capture_words)) != hipSuccess) {
        (void)hipGetLastError();
        return;
    }
    capture_words_ = (unsigned int*)ptr;
}

unsigned int* SideRegistry::debug_word(unsigned int dealing) {
    std::lock_guard<std::mutex> g(mu_);
    if (!capture_words_) return nullptr;
    unsigned int* word = capture_words_ + (kCaptureWords - 1);
    static unsigned int last = ~0u;
    const unsigned int v = 0x80000000u | (dealing & 0xfu);
    if (v != last) {
        DeviceGuard dev(device_);
        if (hipMemcpy(word, &v, sizeof v, hipMemcpyHostToDevice) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
        last = v;
    }
    return word;
}

unsigned int* SideRegistry::capture_word(void* stream, bool* capturing) {
    *capturing = false;
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    unsigned long long id = 0;
    if (hipStreamGetCaptureInfo((hipStream_t)stream, &status, &id) != hipSuccess) {
        (void)hipGetLastError();
        *capturing = true;                           // cannot tell: treat as captured, without a word
        return nullptr;
    }
    if (status == hipStreamCaptureStatusNone) return nullptr;
    *capturing = true;
    if (status != hipStreamCaptureStatusActive) return nullptr;
    std::lock_guard<std::mutex> g(mu_);
    if (!capture_words_) return nullptr;
    const auto key = std::make_pair(id, stream);
    auto it = capture_word_of_.find(key);
    if (it != capture_word_of_.end()) return capture_words_ + it->second;
    if (capture_words_used_ >= kCaptureWords - 1) return nullptr;      // the last word is the A/B switch's
    unsigned int* word = capture_words_ + capture_words_used_;
    DeviceGuard dev(device_);
    hipLaunchKernelGGL(sa_scout, dim3(1), dim3(64), 0, (hipStream_t)stream, word);      // captured, like the launch that follows
    if (hipGetLastError() != hipSuccess) return nullptr;
    capture_word_of_.emplace(key, capture_words_used_++);
    return word;
}

// The pinned words the sided kernels report their XCD to.  Allocated when the device is set up, so
// that a first sided launch may happen under stream capture (which allows no allocation).
bool SideRegistry::ensure_feedback_locked() {
    if (feedback_) return true;
    DeviceGuard dev(device_);
    void* p = nullptr;
    if (hipHostMalloc(&p, kFeedbackSlots * 64, hipHostMallocMapped) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    std::fill_n((unsigned int*)p, kFeedbackSlots * 16, 0u);
    feedback_ = (volatile unsigned int*)p;
    return true;
}

void SideRegistry::init_feedback() {
    std::lock_guard<std::mutex> g(mu_);
    (void)ensure_feedback_locked();
}

// The probe behind sideaware_probe_sides and sideaware_probe_sides_noalloc: everything runs on the
// caller's stream, the results stay on the device.  `work` holds 16 * count + 16 words.
int SideRegistry::probe_on_stream(const void* region, size_t bytes, unsigned long long seed, int count, int* sides,
                                  void* stream, unsigned int* work) {
    DeviceGuard dev(device_);
    hipStream_t st = (hipStream_t)stream;
    const unsigned long long granules = bytes >> kSideGranuleLog2;
    const int words = 16 * count + 16;
    for (int pass = 0; pass < 2; pass++) {
        hipLaunchKernelGGL(sa_side_clear, dim3((words + 255) / 256), dim3(256), 0, st, work, words);
        hipLaunchKernelGGL(sa_side_probe_seeded, dim3(kProbeGroups), dim3(64), 0, st, (const char*)region, granules, seed,
                           count, work);
        if (pass == 0) {
            hipLaunchKernelGGL(sa_side_scrub, dim3(2048), dim3(256), 0, st, (const sa_probe_v4i*)region, kScrubBytes / 16,
                               work + 16 * (size_t)count);
        }
    }
    hipLaunchKernelGGL(sa_side_classify, dim3((count + 63) / 64), dim3(64), 0, st, work, count, sides);
    const hipError_t err = hipGetLastError();
    return err == hipSuccess ? 0 : (int)err;
}

int SideRegistry::probe_sides(const void* region, size_t bytes, unsigned long long seed, int count, int* sides,
                              void* stream, bool allocate) {
    if (!region || !sides || count < 1 || bytes < kScrubBytes || ((uintptr_t)region & ((1u << kSideGranuleLog2) - 1))) return -1;
    if (!allocate) {
        // no allocation of any kind: the device's static array is the work space
        if (count > kNoAllocMaxSamples) return -2;
        unsigned int* work;
        {
            std::lock_guard<std::mutex> g(mu_);
            work = static_scratch_;
        }
        if (!work) return -3;
        return probe_on_stream(region, bytes, seed, count, sides, stream, work);
    }
    DeviceGuard dev(device_);
    hipStream_t st = (hipStream_t)stream;
    unsigned int* work = nullptr;
    const size_t work_bytes = (16 * (size_t)count + 16) * sizeof(unsigned int);
    // stream-ordered work space: allocated and given back in the stream's own order, no host wait
    bool ordered = hipMallocAsync((void**)&work, work_bytes, st) == hipSuccess;
    if (!ordered) {
        (void)hipGetLastError();
        if (hipMalloc((void**)&work, work_bytes) != hipSuccess) {
            (void)hipGetLastError();
            return -4;
        }
    }
    const int rc = probe_on_stream(region, bytes, seed, count, sides, stream, work);
    if (ordered) {
        if (hipFreeAsync(work, st) != hipSuccess) (void)hipGetLastError();
    } else {
        (void)hipStreamSynchronize(st);
        (void)hipFree(work);
    }
    return rc;
}

SideRegistry::~SideRegistry() {
    // device buffers, the stream and the pinned slots live until the process ends: launches that
    // report into the slots may still be queued
}

// Times loads at base + offsets[i] from every XCD and says, for each i, which half of the XCDs is
// nearer: 0 (XCDs 0 .. n/2-1), 1, or -1 when the two halves do not differ clearly.
bool SideRegistry::measure_locked(const char* base, size_t bytes, const std::vector<uint64_t>& offsets, std::vector<int>* sides,
                                  bool busy_device) {
    const int n = (int)offsets.size();
    sides->assign(n, -1);
    if (n == 0 || n > kMaxProbe || bytes < kScrubBytes) return false;
    DeviceGuard dev(device_);
    RelaxedCapture relaxed;
    if (!probe_stream_) {
        hipStream_t s = nullptr;
        if (hipStreamCreateWithFlags(&s, hipStreamNonBlocking) != hipSuccess) { (void)hipGetLastError(); return false; }
        probe_stream_ = s;
        if (hipMalloc((void**)&probe_offsets_, kMaxProbe * sizeof(uint64_t)) != hipSuccess ||
            hipMalloc((void**)&probe_lat_, (16 * kMaxProbe + 16) * sizeof(unsigned int)) != hipSuccess) {
            (void)hipGetLastError();
            return false;
        }
    }
    if (!probe_offsets_ || !probe_lat_) return false;
    hipStream_t st = (hipStream_t)probe_stream_;
    std::vector<unsigned int> lat(16 * (size_t)n);
    bool ok = hipMemcpyAsync(probe_offsets_, offsets.data(), n * sizeof(uint64_t), hipMemcpyHostToDevice, st) == hipSuccess;
    // Two passes with a sweep through the start of the region after each: the first pass brings the
    // sampled lines into the memory-side cache (so the second times the fabric, not DRAM), the
    // sweep pushes them out of the XCDs' own L2s again (which keep clean lines across kernels and
    // would answer the second pass themselves).
    for (int pass = 0; pass < 2 && ok; pass++) {
        ok = hipMemsetAsync(probe_lat_, 0, 16 * (size_t)n * sizeof(unsigned int), st) == hipSuccess;
        if (!ok) break;
        hipLaunchKernelGGL(sa_side_probe, dim3(kProbeGroups), dim3(64), 0, st, base, probe_offsets_, n, probe_lat_);
        if (pass == 0) {
            hipLaunchKernelGGL(sa_side_scrub, dim3(2048), dim3(256), 0, st, (const sa_probe_v4i*)base, kScrubBytes / 16,
                               probe_lat_ + 16 * (size_t)kMaxProbe);
        }
        ok = hipGetLastError() == hipSuccess;
    }
    ok = ok && hipMemcpyAsync(lat.data(), probe_lat_, lat.size() * sizeof(unsigned int), hipMemcpyDeviceToHost, st) == hipSuccess;
    ok = ok && hipStreamSynchronize(st) == hipSuccess;
    if (!ok) { (void)hipGetLastError(); return false; }
    for (int i = 0; i < n; i++) {
        // per half of the device, the middle of its XCDs' times (one XCD delayed by something else
        // then changes nothing)
        unsigned int v[2][kProbeGroups / 2];
        int cnt[2] = {0, 0};
        for (int x = 0; x < kProbeGroups; x++) {
            const unsigned int t = lat[(size_t)x * n + i];
            if (t == 0 || t == ~0u) continue;
            const int h = x / (kProbeGroups / 2);
            v[h][cnt[h]++] = t;
        }
        if (cnt[0] < 3 || cnt[1] < 3) continue;
        double mid[2];
        for (int h = 0; h < 2; h++) {
            std::sort(v[h], v[h] + cnt[h]);
            mid[h] = cnt[h] == 4 ? 0.5 * (v[h][1] + v[h][2]) : v[h][1];
        }
        const double a = mid[0], b = mid[1];
        const double lo = a < b ? a : b, hi = a < b ? b : a;
        // Idle: near about 450 cycles, far about 680: a fifth apart is clear.  With other kernels
        // running both rise (740 / 880): a tenth apart, and at least 60 cycles, still tells the halves
        // apart most of the time, which is good enough for a vote that tolerates a few wrong answers.
        const bool clear = busy_device ? (hi - lo >= 60.0 && hi - lo >= 0.1 * lo) : (hi - lo >= 0.2 * lo);
        if (side_debug() && !clear) {
            std::fprintf(stderr, "sideaware: probe %3d at +0x%llx:", i, (unsigned long long)offsets[i]);
            for (int x = 0; x < kProbeGroups; x++) std::fprintf(stderr, " %u", lat[(size_t)x * n + i]);
            std::fprintf(stderr, "\n");
        }
        if (!clear) continue;
        (*sides)[i] = a < b ? 0 : 1;
    }
    return true;
}

// Which address bits decide the side?  For every candidate bit, a few granules and their partners
// with that bit flipped: a bit is in the hash when (all but at most one of) the pairs land on
// different sides, out of it when (all but at most one) land on the same side, and an attempt fails on
// anything in between.  A failed attempt (timings disturbed by whatever else the device was doing)
// is repeated with other sample granules, a few times; a device that has no such structure fails
// every time and is then treated as one-sided for the life of the process.
void SideRegistry::discover_locked() {
    if (discovered_) return;
    discovered_ = true;
    hash_ = SideHash();
    if (!side_probing_enabled()) return;
    DeviceGuard dev(device_);
    int xcds = 0;
    if (hipDeviceGetAttribute(&xcds, hipDeviceAttributeNumberOfXccs, device_) != hipSuccess || xcds != kProbeGroups) {
        (void)hipGetLastError();
        if (side_debug()) std::fprintf(stderr, "sideaware: side discovery: %d XCDs, need %d\n", xcds, kProbeGroups);
        return;
    }
    constexpr size_t kBytes = 1ull << 30;
    constexpr int kLowBit = 12, kHighBit = 29, kPairsPerBit = 8, kPairsNeeded = 5, kAttempts = 3;
    size_t free_bytes = 0, total = 0;
    if (hipMemGetInfo(&free_bytes, &total) != hipSuccess || free_bytes < 2 * kBytes) { (void)hipGetLastError(); return; }
    char* scratch = nullptr;
    if (hipMalloc((void**)&scratch, kBytes) != hipSuccess) { (void)hipGetLastError(); return; }
    uint64_t lcg = 0x9e3779b97f4a7c15ull;
    for (int attempt = 1; attempt <= kAttempts && !hash_.known; attempt++) {
        std::vector<uint64_t> offsets;
        for (int b = kLowBit; b <= kHighBit; b++) {
            for (int j = 0; j < kPairsPerBit; j++) {
                lcg = lcg * 6364136223846793005ull + 1442695040888963407ull;
                uint64_t x = (lcg >> 20) % kBytes;
                x &= ~((1ull << kLowBit) - 1) & ~(1ull << b);
                offsets.push_back(x);
                offsets.push_back(x | (1ull << b));
            }
        }
        std::vector<int> sides;
        if (!measure_locked(scratch, kBytes, offsets, &sides, /*busy_device=*/false)) {
            if (side_debug()) std::fprintf(stderr, "sideaware: side discovery: the probe could not run\n");
            break;
        }
        uint64_t mask = 0;
        size_t at = 0;
        bool consistent = true;
        for (int b = kLowBit; b <= kHighBit; b++) {
            int flips = 0, same = 0;
            for (int j = 0; j < kPairsPerBit; j++, at += 2) {
                if (sides[at] < 0 || sides[at + 1] < 0) continue;
                (sides[at] != sides[at + 1] ? flips : same)++;
            }
            if (side_debug()) {
                std::fprintf(stderr, "sideaware: side discovery, attempt %d: bit %d: %d pairs flip, %d do not\n", attempt, b,
                             flips, same);
            }
            if (flips >= kPairsNeeded && same <= 1) mask |= 1ull << b;
            else if (!(same >= kPairsNeeded && flips <= 1)) consistent = false;      // not a parity of address bits
        }
        // the kernels assume granules of exactly 8 KiB
        if (!consistent || !((mask >> kSideGranuleLog2) & 1) || (mask & ((1ull << kSideGranuleLog2) - 1))) continue;
        hash_.known = true;
        hash_.address_mask = mask;
    }
    (void)hipFree(scratch);
}

void SideRegistry::discover() {
    std::lock_guard<std::mutex> g(mu_);
    discover_locked();
}

// The arena's constant: a vote over granules spread across it.  A few samples may go the other way
// (a timing that went wrong, or a stretch of the arena that is not physically contiguous with the
// rest: there the sided map is simply wrong, which costs speed, not results); more than a few mean
// the arena is not laid out as the hash says.  Too few clear samples (the device was busy with
// other work while the probe ran) leave the arena unknown for now: a later lookup tries again.
void SideRegistry::vote_locked(ArenaSide& a) {
    a.tries++;
    if (!hash_.known || a.bytes < (1u << kSidePairLog2) || a.base % (1u << kSidePairLog2) != 0) return;
    constexpr int kSamples = 192;
    std::vector<uint64_t> offsets;
    uint64_t lcg = 0x2545f4914f6cdd1dull ^ (uint64_t)a.base ^ ((uint64_t)a.tries << 40);
    const uint64_t granules = a.bytes >> kSideGranuleLog2;
    for (int i = 0; i < kSamples; i++) {
        lcg = lcg * 6364136223846793005ull + 1442695040888963407ull;
        const uint64_t gi = i < 8 ? (uint64_t)i * 37 % granules : (lcg >> 17) % granules;
        offsets.push_back(gi << kSideGranuleLog2);
    }
    std::vector<int> sides;
    if (!measure_locked((const char*)a.base, a.bytes, offsets, &sides, /*busy_device=*/true)) return;
    int votes[2] = {0, 0};
    for (int i = 0; i < kSamples; i++) {
        if (sides[i] < 0) continue;
        votes[(unsigned)sides[i] ^ side_parity(offsets[i] & hash_.address_mask)]++;
    }
    const int valid = votes[0] + votes[1];
    if (side_debug()) std::fprintf(stderr, "sideaware: arena %p (%zu MiB), try %d: votes %d / %d\n", (void*)a.base, a.bytes >> 20, a.tries, votes[0], votes[1]);
    const int minority = votes[0] < votes[1] ? votes[0] : votes[1];
    if (valid >= kSamples / 2) {
        if (minority * 32 <= valid) {
            a.known = true;
            a.flip = votes[1] > votes[0] ? 1u : 0u;
        } else {
            a.tries = kMaxVoteTries;                 // clearly measured, clearly not laid out as the hash says
        }
    }
}

bool SideRegistry::add_arena(void* base, size_t bytes) {
    std::lock_guard<std::mutex> g(mu_);
    discover_locked();
    ArenaSide a;
    a.base = (uintptr_t)base;
    a.bytes = bytes;
    for (const ArenaSide& other : arenas_) {
        if (a.base < other.base + other.bytes && other.base < a.base + a.bytes) return false;   // overlaps a known one
    }
    vote_locked(a);
    arenas_.push_back(a);
    return a.known;
}

// An arena whose vote was inconclusive is measured again when the pool next places a region in
// it (an allocation that carves is a slow path already; launches never wait for a probe), a few
// times at most and not on every placement.
void SideRegistry::maybe_vote_again_locked(ArenaSide& a) {
    if (a.known || a.tries >= kMaxVoteTries) return;
    if (++a.asked % 4 != 0) return;
    vote_locked(a);
}

void SideRegistry::remove_arena(void* base) {
    std::lock_guard<std::mutex> g(mu_);
    for (size_t i = 0; i < arenas_.size(); i++) {
        if (arenas_[i].base == (uintptr_t)base) {
            arenas_[i] = arenas_.back();
            arenas_.pop_back();
            return;
        }
    }
}

SideHash SideRegistry::hash() {
    std::lock_guard<std::mutex> g(mu_);
    return hash_;
}

int SideRegistry::arenas_known() {
    std::lock_guard<std::mutex> g(mu_);
    int n = 0;
    for (const ArenaSide& a : arenas_) n += a.known ? 1 : 0;
    return n;
}

bool SideRegistry::lookup(const void* addr, size_t bytes, SideMap* out) {
    const uintptr_t p = (uintptr_t)addr;
    std::lock_guard<std::mutex> g(mu_);
    if (!hash_.known) return false;
    for (const ArenaSide& a : arenas_) {
        if (p >= a.base && p - a.base < a.bytes) {
            if (!a.known || bytes > a.bytes - (p - a.base)) return false;
            out->origin_address = a.base;
            out->pair_mask = hash_.pair_mask();
            out->flip = a.flip;
            return true;
        }
    }
    return false;
}

bool SideRegistry::arena_of(const void* addr, uintptr_t* base, unsigned int* flip, bool placing) {
    const uintptr_t p = (uintptr_t)addr;
    std::lock_guard<std::mutex> g(mu_);
    if (!hash_.known) return false;
    for (ArenaSide& a : arenas_) {
        if (p >= a.base && p - a.base < a.bytes) {
            if (placing) maybe_vote_again_locked(a);
            if (!a.known) return false;
            *base = a.base;
            *flip = a.flip;
            return true;
        }
    }
    return false;
}

int SideRegistry::side_of(const void* addr) {
    uintptr_t base = 0;
    unsigned int flip = 0;
    if (!arena_of(addr, &base, &flip)) return -1;
    const SideHash h = hash();
    return (int)(side_parity(((uintptr_t)addr - base) & h.address_mask) ^ flip);
}

int SideRegistry::slot_of_locked(void* stream) {
    auto it = slot_of_stream_.find(stream);
    if (it != slot_of_stream_.end()) return it->second;
    // more streams than slots: the late ones share the last slot (and each other's reports)
    const int slot = (int)slot_of_stream_.size() < kFeedbackSlots ? (int)slot_of_stream_.size() : kFeedbackSlots - 1;
    slot_of_stream_.emplace(stream, slot);
    return slot;
}

unsigned int* SideRegistry::feedback_slot(void* stream, unsigned int* dealing, bool account) {
    std::lock_guard<std::mutex> g(mu_);
    *dealing = 0;
    if (!ensure_feedback_locked()) return nullptr;
    const int slot = slot_of_locked(stream);
    volatile unsigned int* word = feedback_ + (size_t)slot * 16;
    const unsigned int v = *word;
    if (v & 0x80000000u) {
        SlotState& st = slot_state_[slot];
        const unsigned int k = v & 0xfu;
        *dealing = k;
        if (account) {
            if (st.has && k != st.believed) st.flaps = st.flaps + 4 > 32 ? 32 : st.flaps + 4;
            else if (st.flaps > 0) st.flaps--;
            st.believed = k;
            st.has = true;
        }
    }
    return (unsigned int*)word;
}

bool SideRegistry::stream_is_steady(void* stream) {
    std::lock_guard<std::mutex> g(mu_);
    auto it = slot_of_stream_.find(stream);
    if (it == slot_of_stream_.end()) return true;
    SlotState& st = slot_state_[it->second];
    if (st.flaps < kUnsteadyFlaps) return true;
    st.flaps--;                                      // this launch goes striped; a few of those and sided is tried again
    return false;
}

void SideRegistry::report_dealing(void* stream, unsigned int dealing) {
    std::lock_guard<std::mutex> g(mu_);
    if (!ensure_feedback_locked()) return;
    volatile unsigned int* word = feedback_ + (size_t)slot_of_locked(stream) * 16;
    *word = 0x80000000u | (dealing & 0xfu);
}

}  // namespace sideaware
