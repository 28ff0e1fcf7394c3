// bench_ceiling_kernels.so: framework-free streaming kernels for gfx950 that measure what the memory system of
// an MI355X delivers to the simplest possible read, write and copy loops.  They share nothing with
// the elementwise template (no op hooks, no launch planner): `bench.py --ceiling` times them beside
// the library's own kernels so that "the hardware tops out here" is a measurement, not a claim.
//
// Every kernel moves 16-byte vectors; a wave instruction covers 1 KiB of consecutive addresses
// unless the lane-contiguous flag is set.  Sizes must be whole numbers of tiles: the host checks.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>

typedef int v4i __attribute__((ext_vector_type(4)));

enum : int {
    kNtLoads = 1,          // loads carry the nontemporal hint
    kNtStores = 2,         // stores carry the nontemporal hint
    kLaneContiguous = 4,   // a lane takes K consecutive vectors instead of K vectors a block apart
    kWaitStores = 8,       // persistent kernels: stores are acknowledged before the next loads are issued
    kPrefetch = 16,        // persistent copies: the next chunk's loads are issued before this chunk's stores
    kSplitRoles = 32,      // tile kernel: workgroup pairs alternate between reading src and filling dst
};

template <bool NT>
__device__ __forceinline__ v4i ld(const v4i* p) {
    return NT ? __builtin_nontemporal_load(p) : *p;
}
template <bool NT>
__device__ __forceinline__ void st(v4i* p, v4i v) {
    if (NT) __builtin_nontemporal_store(v, p); else *p = v;
}

__device__ __forceinline__ void sink_if_magic(v4i acc, int* sink) {
    // keeps the loads alive: the data is random, so four equal words of this value never occur
    if ((acc.x ^ acc.y) == 0x5a5a5a5a && (acc.z ^ acc.w) == 0x5a5a5a5a && acc.x == acc.z) sink[0] = 1;
}

// XCD-striped tile number of a workgroup: workgroups are dealt to the 8 XCDs in turn, so the
// workgroup with index b runs on XCD b % 8; stripe s (2^r tiles) of the array goes to XCD s % 8.
__device__ __forceinline__ long long striped_tile(unsigned b, unsigned r) {
    const unsigned xcd = b & 7u, slot = b >> 3;
    return ((((long long)(slot >> r) << 3) + xcd) << r) + (slot & ((1u << r) - 1u));
}

// One workgroup per tile of K * blockDim.x vectors.  dst == nullptr: read only; src == nullptr:
// write only; both: copy (dst == src: read-modify-write in place).
// `stamps` (optional): two device words per workgroup, into which it writes the device clock at
// its start and at its end (after its stores were acknowledged), so the host can see when each
// XCD started and finished its share of a launch.
template <int K, bool NTL, bool NTS, bool CONTIG>
__global__ __launch_bounds__(1024) void tile_kernel(v4i* dst, const v4i* src, unsigned r, int flags, int* sink,
                                                    unsigned long long* stamps) {
    if (stamps && threadIdx.x == 0) stamps[2 * (size_t)blockIdx.x] = wall_clock64();
    const unsigned B = blockDim.x, tid = threadIdx.x;
    const long long tile = striped_tile(blockIdx.x, r);
    const long long base = tile * (long long)(B * K);
    bool do_read = src != nullptr, do_write = dst != nullptr;
    if (flags & kSplitRoles) {
        // independent streams: half of the workgroups only read, the other half only write
        const bool reader = ((blockIdx.x >> 3) & 1u) == 0;
        do_read = reader;
        do_write = !reader;
    }
    v4i v[K];
    if (do_read) {
        #pragma unroll
        for (int k = 0; k < K; k++) {
            const long long i = CONTIG ? base + (long long)tid * K + k : base + (long long)k * B + tid;
            v[k] = ld<NTL>(src + i);
        }
    } else {
        #pragma unroll
        for (int k = 0; k < K; k++) v[k] = (v4i){(int)tid, k, (int)blockIdx.x, 7};
    }
    if (do_write) {
        #pragma unroll
        for (int k = 0; k < K; k++) {
            const long long i = CONTIG ? base + (long long)tid * K + k : base + (long long)k * B + tid;
            st<NTS>(dst + i, v[k]);
        }
    } else {
        v4i acc = v[0];
        #pragma unroll
        for (int k = 1; k < K; k++) acc ^= v[k];
        sink_if_magic(acc, sink);
    }
    if (stamps && threadIdx.x == 0) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");          // this wave's stores are acknowledged
        stamps[2 * (size_t)blockIdx.x + 1] = wall_clock64();
    }
}

// The one-workgroup-per-4-KiB kernel with the cache-policy bits of its loads and stores spelled out
// in the instruction (sc0 / sc1: the scope the access is coherent at, workgroup / agent / both:
// system; nt: nontemporal).  mode 0: copy, 1: read only, 2: write only.
#define POLICY_KERNEL(NAME, LOADP, STOREP)                                                                   \
    __global__ __launch_bounds__(256) void NAME(v4i* dst, const v4i* src, unsigned r, int mode, int* sink) {  \
        const long long i = striped_tile(blockIdx.x, r) * 256 + threadIdx.x;                                  \
        v4i v = (v4i){(int)threadIdx.x, 1, (int)blockIdx.x, 7};                                               \
        if (mode != 2) {                                                                                      \
            const v4i* p = src + i;                                                                           \
            asm volatile("global_load_dwordx4 %0, %1, off " LOADP "\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory"); \
        }                                                                                                     \
        if (mode != 1) {                                                                                      \
            v4i* q = dst + i;                                                                                 \
            asm volatile("global_store_dwordx4 %0, %1, off " STOREP "\n\ts_nop 1" : : "v"(q), "v"(v) : "memory"); \
        } else {                                                                                              \
            sink_if_magic(v, sink);                                                                           \
        }                                                                                                     \
    }
POLICY_KERNEL(policy_plain_plain, "", "")
POLICY_KERNEL(policy_plain_nt, "", "nt")
POLICY_KERNEL(policy_plain_sc1, "", "sc1")
POLICY_KERNEL(policy_plain_sc0sc1, "", "sc0 sc1")
POLICY_KERNEL(policy_plain_sc1nt, "", "sc1 nt")
POLICY_KERNEL(policy_plain_sc0sc1nt, "", "sc0 sc1 nt")
POLICY_KERNEL(policy_plain_sc0, "", "sc0")
POLICY_KERNEL(policy_nt_plain, "nt", "")
POLICY_KERNEL(policy_nt_nt, "nt", "nt")
POLICY_KERNEL(policy_nt_sc1, "nt", "sc1")
POLICY_KERNEL(policy_nt_sc0sc1, "nt", "sc0 sc1")
POLICY_KERNEL(policy_nt_sc1nt, "nt", "sc1 nt")
POLICY_KERNEL(policy_nt_sc0sc1nt, "nt", "sc0 sc1 nt")
POLICY_KERNEL(policy_nt_sc0, "nt", "sc0")
POLICY_KERNEL(policy_sc1_plain, "sc1", "")
POLICY_KERNEL(policy_sc1_nt, "sc1", "nt")
POLICY_KERNEL(policy_sc1_sc1, "sc1", "sc1")
POLICY_KERNEL(policy_sc1_sc0sc1, "sc1", "sc0 sc1")
POLICY_KERNEL(policy_sc1_sc1nt, "sc1", "sc1 nt")
POLICY_KERNEL(policy_sc1_sc0sc1nt, "sc1", "sc0 sc1 nt")
POLICY_KERNEL(policy_sc1_sc0, "sc1", "sc0")
POLICY_KERNEL(policy_sc0sc1_plain, "sc0 sc1", "")
POLICY_KERNEL(policy_sc0sc1_nt, "sc0 sc1", "nt")
POLICY_KERNEL(policy_sc0sc1_sc1, "sc0 sc1", "sc1")
POLICY_KERNEL(policy_sc0sc1_sc0sc1, "sc0 sc1", "sc0 sc1")
POLICY_KERNEL(policy_sc0sc1_sc1nt, "sc0 sc1", "sc1 nt")
POLICY_KERNEL(policy_sc0sc1_sc0sc1nt, "sc0 sc1", "sc0 sc1 nt")
POLICY_KERNEL(policy_sc0sc1_sc0, "sc0 sc1", "sc0")
POLICY_KERNEL(policy_sc1nt_plain, "sc1 nt", "")
POLICY_KERNEL(policy_sc1nt_nt, "sc1 nt", "nt")
POLICY_KERNEL(policy_sc1nt_sc1, "sc1 nt", "sc1")
POLICY_KERNEL(policy_sc1nt_sc0sc1, "sc1 nt", "sc0 sc1")
POLICY_KERNEL(policy_sc1nt_sc1nt, "sc1 nt", "sc1 nt")
POLICY_KERNEL(policy_sc1nt_sc0sc1nt, "sc1 nt", "sc0 sc1 nt")
POLICY_KERNEL(policy_sc1nt_sc0, "sc1 nt", "sc0")
POLICY_KERNEL(policy_sc0sc1nt_plain, "sc0 sc1 nt", "")
POLICY_KERNEL(policy_sc0sc1nt_nt, "sc0 sc1 nt", "nt")
POLICY_KERNEL(policy_sc0sc1nt_sc1, "sc0 sc1 nt", "sc1")
POLICY_KERNEL(policy_sc0sc1nt_sc0sc1, "sc0 sc1 nt", "sc0 sc1")
POLICY_KERNEL(policy_sc0sc1nt_sc1nt, "sc0 sc1 nt", "sc1 nt")
POLICY_KERNEL(policy_sc0sc1nt_sc0sc1nt, "sc0 sc1 nt", "sc0 sc1 nt")
POLICY_KERNEL(policy_sc0sc1nt_sc0, "sc0 sc1 nt", "sc0")
POLICY_KERNEL(policy_sc0_plain, "sc0", "")
POLICY_KERNEL(policy_sc0_nt, "sc0", "nt")
POLICY_KERNEL(policy_sc0_sc1, "sc0", "sc1")
POLICY_KERNEL(policy_sc0_sc0sc1, "sc0", "sc0 sc1")
POLICY_KERNEL(policy_sc0_sc1nt, "sc0", "sc1 nt")
POLICY_KERNEL(policy_sc0_sc0sc1nt, "sc0", "sc0 sc1 nt")
POLICY_KERNEL(policy_sc0_sc0, "sc0", "sc0")

typedef void (*policy_fn)(v4i*, const v4i*, unsigned, int, int*);
static const struct { const char* loads; const char* stores; policy_fn fn; } kPolicyKernels[] = {
    {"", "", policy_plain_plain},
    {"", "nt", policy_plain_nt},
    {"", "sc1", policy_plain_sc1},
    {"", "sc0 sc1", policy_plain_sc0sc1},
    {"", "sc1 nt", policy_plain_sc1nt},
    {"", "sc0 sc1 nt", policy_plain_sc0sc1nt},
    {"", "sc0", policy_plain_sc0},
    {"nt", "", policy_nt_plain},
    {"nt", "nt", policy_nt_nt},
    {"nt", "sc1", policy_nt_sc1},
    {"nt", "sc0 sc1", policy_nt_sc0sc1},
    {"nt", "sc1 nt", policy_nt_sc1nt},
    {"nt", "sc0 sc1 nt", policy_nt_sc0sc1nt},
    {"nt", "sc0", policy_nt_sc0},
    {"sc1", "", policy_sc1_plain},
    {"sc1", "nt", policy_sc1_nt},
    {"sc1", "sc1", policy_sc1_sc1},
    {"sc1", "sc0 sc1", policy_sc1_sc0sc1},
    {"sc1", "sc1 nt", policy_sc1_sc1nt},
    {"sc1", "sc0 sc1 nt", policy_sc1_sc0sc1nt},
    {"sc1", "sc0", policy_sc1_sc0},
    {"sc0 sc1", "", policy_sc0sc1_plain},
    {"sc0 sc1", "nt", policy_sc0sc1_nt},
    {"sc0 sc1", "sc1", policy_sc0sc1_sc1},
    {"sc0 sc1", "sc0 sc1", policy_sc0sc1_sc0sc1},
    {"sc0 sc1", "sc1 nt", policy_sc0sc1_sc1nt},
    {"sc0 sc1", "sc0 sc1 nt", policy_sc0sc1_sc0sc1nt},
    {"sc0 sc1", "sc0", policy_sc0sc1_sc0},
    {"sc1 nt", "", policy_sc1nt_plain},
    {"sc1 nt", "nt", policy_sc1nt_nt},
    {"sc1 nt", "sc1", policy_sc1nt_sc1},
    {"sc1 nt", "sc0 sc1", policy_sc1nt_sc0sc1},
    {"sc1 nt", "sc1 nt", policy_sc1nt_sc1nt},
    {"sc1 nt", "sc0 sc1 nt", policy_sc1nt_sc0sc1nt},
    {"sc1 nt", "sc0", policy_sc1nt_sc0},
    {"sc0 sc1 nt", "", policy_sc0sc1nt_plain},
    {"sc0 sc1 nt", "nt", policy_sc0sc1nt_nt},
    {"sc0 sc1 nt", "sc1", policy_sc0sc1nt_sc1},
    {"sc0 sc1 nt", "sc0 sc1", policy_sc0sc1nt_sc0sc1},
    {"sc0 sc1 nt", "sc1 nt", policy_sc0sc1nt_sc1nt},
    {"sc0 sc1 nt", "sc0 sc1 nt", policy_sc0sc1nt_sc0sc1nt},
    {"sc0 sc1 nt", "sc0", policy_sc0sc1nt_sc0},
    {"sc0", "", policy_sc0_plain},
    {"sc0", "nt", policy_sc0_nt},
    {"sc0", "sc1", policy_sc0_sc1},
    {"sc0", "sc0 sc1", policy_sc0_sc0sc1},
    {"sc0", "sc1 nt", policy_sc0_sc1nt},
    {"sc0", "sc0 sc1 nt", policy_sc0_sc0sc1nt},
    {"sc0", "sc0", policy_sc0_sc0},
};

// The one-workgroup-per-4-KiB nt copy with unequal shares per XCD.  Workgroups are dealt to the
// XCDs in turn, so each XCD gets the same number of workgroup slots (own + the largest extra);
// XCD x does only the first cut[x] of its own tiles, and the tiles the donors leave over are done
// by the helper slots (slot >= own) of the XCDs with extra[x] > 0, in donor order.
struct xcd_shares {
    int cut[8];
    int extra[8];
};
__global__ __launch_bounds__(256) void balanced_copy_kernel(v4i* dst, const v4i* src, unsigned r, int own, xcd_shares sh,
                                                            unsigned long long* stamps) {
    const unsigned tid = threadIdx.x, xcd = blockIdx.x & 7u;
    int slot = (int)(blockIdx.x >> 3);
    if (stamps && tid == 0) stamps[2 * (size_t)blockIdx.x] = wall_clock64();
    unsigned owner = xcd;
    if (slot >= own) {
        int h = slot - own;
        if (h >= sh.extra[xcd]) return;
        for (unsigned y = 0; y < xcd; y++) h += sh.extra[y];          // position in the list of donated tiles
        owner = 8;
        for (unsigned d = 0; d < 8; d++) {
            const int given = own - sh.cut[d];
            if (owner == 8 && h < given) { owner = d; slot = sh.cut[d] + h; }
            if (owner == 8) h -= given;
        }
        if (owner == 8) return;
    } else if (slot >= sh.cut[xcd]) {
        return;                                                       // donated away
    }
    const unsigned uslot = (unsigned)slot;
    const long long tile = ((((long long)(uslot >> r) << 3) + owner) << r) + (uslot & ((1u << r) - 1u));
    const long long i = tile * 256 + tid;
    const v4i v = ld<true>(src + i);
    st<true>(dst + i, v);
    if (stamps && tid == 0) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        stamps[2 * (size_t)blockIdx.x + 1] = wall_clock64();
    }
}

// A fixed grid; workgroup b takes chunks b, b + grid, b + 2 grid, ... of K * blockDim.x vectors
// (dst == nullptr: read only; src == nullptr: write only).
// All K loads of a chunk are complete before its first store is issued, so each workgroup
// alternates between a read burst and a write burst.  With period_ticks != 0 every wave waits for
// the next multiple of period_ticks of the device's 100 MHz constant clock before each read
// burst: the bursts of all workgroups of the chip then line up, and the memory sees alternating
// read-mostly and write-mostly phases instead of a steady mix.
template <int K, bool NTL, bool NTS>
__global__ __launch_bounds__(1024) void persistent_kernel(v4i* dst, const v4i* src, long long n_chunks, int flags,
                                                          unsigned period_ticks, int* sink) {
    const unsigned B = blockDim.x, tid = threadIdx.x;
    const long long chunk = (long long)B * K;
    for (long long c = blockIdx.x; c < n_chunks; c += gridDim.x) {
        if (period_ticks) {
            const unsigned long long t = wall_clock64();
            const unsigned long long target = (t / period_ticks + 1) * period_ticks;
            while (wall_clock64() < target) __builtin_amdgcn_s_sleep(2);
        }
        const long long base = c * chunk + tid;
        v4i v[K];
        if (src) {
            #pragma unroll
            for (int k = 0; k < K; k++) v[k] = ld<NTL>(src + base + (long long)k * B);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        } else {
            #pragma unroll
            for (int k = 0; k < K; k++) v[k] = (v4i){(int)tid, k, (int)c, 7};
        }
        if (dst) {
            #pragma unroll
            for (int k = 0; k < K; k++) st<NTS>(dst + base + (long long)k * B, v[k]);
            if (flags & kWaitStores) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        } else {
            v4i acc = v[0];
            #pragma unroll
            for (int k = 1; k < K; k++) acc ^= v[k];
            sink_if_magic(acc, sink);
        }
    }
}

// The same fixed grid for a copy, software-pipelined: the loads of a workgroup's next chunk are in
// flight while the current chunk is stored, so a workgroup always has reads and writes outstanding
// instead of alternating between them.
template <int K, bool NTL, bool NTS>
__global__ __launch_bounds__(1024) void persistent_prefetch_kernel(v4i* dst, const v4i* src, long long n_chunks, int flags,
                                                                   unsigned period_ticks, int* sink) {
    const unsigned B = blockDim.x, tid = threadIdx.x;
    const long long chunk = (long long)B * K;
    long long c = blockIdx.x;
    if (c >= n_chunks) return;
    v4i cur[K], nxt[K];
    #pragma unroll
    for (int k = 0; k < K; k++) cur[k] = ld<NTL>(src + c * chunk + tid + (long long)k * B);
    for (;;) {
        const long long cn = c + gridDim.x;
        const bool more = cn < n_chunks;                       // uniform across the workgroup
        if (more) {
            #pragma unroll
            for (int k = 0; k < K; k++) nxt[k] = ld<NTL>(src + cn * chunk + tid + (long long)k * B);
        }
        #pragma unroll
        for (int k = 0; k < K; k++) st<NTS>(dst + c * chunk + tid + (long long)k * B, cur[k]);
        if (!more) break;
        #pragma unroll
        for (int k = 0; k < K; k++) cur[k] = nxt[k];
        c = cn;
    }
}

typedef void (*tile_fn)(v4i*, const v4i*, unsigned, int, int*, unsigned long long*);
typedef void (*persistent_fn)(v4i*, const v4i*, long long, int, unsigned, int*);

template <int K>
static tile_fn pick_tile(int flags) {
    const bool c = flags & kLaneContiguous;
    switch (flags & 3) {
        case 0: return c ? tile_kernel<K, false, false, true> : tile_kernel<K, false, false, false>;
        case 1: return c ? tile_kernel<K, true, false, true> : tile_kernel<K, true, false, false>;
        case 2: return c ? tile_kernel<K, false, true, true> : tile_kernel<K, false, true, false>;
        default: return c ? tile_kernel<K, true, true, true> : tile_kernel<K, true, true, false>;
    }
}

template <int K>
static persistent_fn pick_persistent(int flags) {
    if (flags & kPrefetch) {
        switch (flags & 3) {
            case 0: return persistent_prefetch_kernel<K, false, false>;
            case 1: return persistent_prefetch_kernel<K, true, false>;
            case 2: return persistent_prefetch_kernel<K, false, true>;
            default: return persistent_prefetch_kernel<K, true, true>;
        }
    }
    switch (flags & 3) {
        case 0: return persistent_kernel<K, false, false>;
        case 1: return persistent_kernel<K, true, false>;
        case 2: return persistent_kernel<K, false, true>;
        default: return persistent_kernel<K, true, true>;
    }
}

static char g_error[256] = "";

static int fail(const char* what) {
    std::snprintf(g_error, sizeof g_error, "%s", what);
    return 1;
}

#pragma GCC visibility push(default)
extern "C" {

const char* hbm_ceiling_last_error(void) { return g_error; }

// One workgroup per tile.  `bytes` must be a multiple of 8 * (k * block * 16) << stripe_log2.
// `stamps`: null, or two device words per tile that receive each workgroup's start and end time.
// Returns 0 when the kernel was launched.
int hbm_ceiling_tile(void* dst, const void* src, size_t bytes, int k, int block, int stripe_log2, int flags,
                     int* sink, unsigned long long* stamps, hipStream_t stream) {
    if (block < 64 || block > 1024 || (block & (block - 1))) return fail("block must be a power of two in 64..1024");
    if (stripe_log2 < 0 || stripe_log2 > 12) return fail("stripe_log2 must be in 0..12");
    if (!dst && !src) return fail("nothing to do");
    if ((flags & kSplitRoles) && (!dst || !src)) return fail("split roles needs both buffers");
    if (!sink) return fail("sink must point at four bytes of device memory");
    const size_t tile_bytes = (size_t)k * block * 16;
    const size_t period = (tile_bytes * 8) << stripe_log2;
    if (bytes == 0 || bytes % period) return fail("bytes must be a whole number of 8-XCD stripe periods");
    const size_t tiles = bytes / tile_bytes;
    if (tiles > 0x7fffffffull) return fail("too many tiles for one grid");
    tile_fn fn = nullptr;
    switch (k) {
        case 1: fn = pick_tile<1>(flags); break;
        case 2: fn = pick_tile<2>(flags); break;
        case 4: fn = pick_tile<4>(flags); break;
        case 8: fn = pick_tile<8>(flags); break;
        case 16: fn = pick_tile<16>(flags); break;
        default: return fail("k must be 1, 2, 4, 8 or 16");
    }
    hipLaunchKernelGGL(fn, dim3((unsigned)tiles), dim3(block), 0, stream, (v4i*)dst, (const v4i*)src,
                       (unsigned)stripe_log2, flags, sink, stamps);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : fail(hipGetErrorString(e));
}

// One workgroup per 4 KiB with the given cache-policy bits on loads and stores ("", "nt", "sc1",
// "sc0 sc1", "sc1 nt", "sc0 sc1 nt", "sc0").  mode 0: copy, 1: read only, 2: write only.
int hbm_ceiling_policy(void* dst, const void* src, size_t bytes, int stripe_log2, const char* loads, const char* stores,
                       int mode, int* sink, hipStream_t stream) {
    if (stripe_log2 < 0 || stripe_log2 > 12) return fail("stripe_log2 must be in 0..12");
    if (!loads || !stores || !sink || mode < 0 || mode > 2) return fail("bad argument");
    if ((mode != 2 && !src) || (mode != 1 && !dst)) return fail("null buffer");
    const size_t period = ((size_t)4096 * 8) << stripe_log2;
    if (bytes == 0 || bytes % period || bytes / 4096 > 0x7fffffffull) return fail("bytes must be a whole number of 8-XCD stripe periods");
    for (const auto& k : kPolicyKernels) {
        if (std::strcmp(k.loads, loads) == 0 && std::strcmp(k.stores, stores) == 0) {
            hipLaunchKernelGGL(k.fn, dim3((unsigned)(bytes / 4096)), dim3(256), 0, stream, (v4i*)dst, (const v4i*)src,
                               (unsigned)stripe_log2, mode, sink);
            hipError_t e = hipGetLastError();
            return e == hipSuccess ? 0 : fail(hipGetErrorString(e));
        }
    }
    return fail("no kernel with these policy bits");
}

// The nt copy, one workgroup per 4 KiB, with per-XCD shares: XCD x does cut[x] of its own tiles plus
// extra[x] of the tiles the others leave over (the sum of own - cut must equal the sum of extra).
// `stamps`: null, or two device words per workgroup slot of the grid, 8 * (own + max extra).
int hbm_ceiling_balanced_copy(void* dst, const void* src, size_t bytes, int stripe_log2, const int* cut, const int* extra,
                              unsigned long long* stamps, hipStream_t stream) {
    if (stripe_log2 < 0 || stripe_log2 > 12) return fail("stripe_log2 must be in 0..12");
    if (!dst || !src || !cut || !extra) return fail("null argument");
    const size_t period = ((size_t)4096 * 8) << stripe_log2;
    if (bytes == 0 || bytes % period) return fail("bytes must be a whole number of 8-XCD stripe periods");
    const long long own = (long long)(bytes / 4096 / 8);
    xcd_shares sh;
    long long given = 0, taken = 0, most = 0;
    for (int x = 0; x < 8; x++) {
        if (cut[x] < 0 || cut[x] > own || extra[x] < 0 || (extra[x] > 0 && cut[x] != own)) return fail("bad shares");
        sh.cut[x] = cut[x];
        sh.extra[x] = extra[x];
        given += own - cut[x];
        taken += extra[x];
        most = extra[x] > most ? extra[x] : most;
    }
    if (given != taken) return fail("donated and taken tiles differ");
    if ((own + most) * 8 > 0x7fffffffll) return fail("too many workgroups");
    hipLaunchKernelGGL(balanced_copy_kernel, dim3((unsigned)((own + most) * 8)), dim3(256), 0, stream, (v4i*)dst,
                       (const v4i*)src, (unsigned)stripe_log2, (int)own, sh, stamps);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : fail(hipGetErrorString(e));
}

// A fixed grid of `grid` workgroups.  `bytes` must be a multiple of k * block * 16.
int hbm_ceiling_persistent(void* dst, const void* src, size_t bytes, int k, int block, int grid, int flags,
                           unsigned period_ticks, int* sink, hipStream_t stream) {
    if (block < 64 || block > 1024 || (block & (block - 1))) return fail("block must be a power of two in 64..1024");
    if (grid < 1 || grid > (1 << 20)) return fail("grid out of range");
    if (!dst && !src) return fail("nothing to do");
    if ((flags & kPrefetch) && (!dst || !src || period_ticks)) return fail("prefetch is for plain copies");
    if ((flags & kPrefetch) && k > 8) return fail("prefetch: k at most 8");
    if (!sink) return fail("sink must point at four bytes of device memory");
    const size_t chunk_bytes = (size_t)k * block * 16;
    if (bytes == 0 || bytes % chunk_bytes) return fail("bytes must be a whole number of chunks");
    persistent_fn fn = nullptr;
    switch (k) {
        case 1: fn = pick_persistent<1>(flags); break;
        case 2: fn = pick_persistent<2>(flags); break;
        case 4: fn = pick_persistent<4>(flags); break;
        case 8: fn = pick_persistent<8>(flags); break;
        case 16: fn = pick_persistent<16>(flags); break;
        case 24: fn = pick_persistent<24>(flags); break;
        default: return fail("k must be 1, 2, 4, 8, 16 or 24");
    }
    hipLaunchKernelGGL(fn, dim3((unsigned)grid), dim3(block), 0, stream, (v4i*)dst, (const v4i*)src,
                       (long long)(bytes / chunk_bytes), flags, period_ticks, sink);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : fail(hipGetErrorString(e));
}

}  // extern "C"
#pragma GCC visibility pop
