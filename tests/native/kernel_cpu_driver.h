// Appended after the kernel template: runs the whole grid on the CPU, lane by lane, and checks
// the result.  stdin carries one case per line:
// "grid num_vectors base_offset_bytes stripe_log2 slot_run [segments]".  With segments > 1 the
// array is cut into that many pieces at arbitrary vector boundaries and all of them go through the
// batched entry point in one grid (only meaningful for ops that do not look at the element index).
//
// Every array is a posix_memalign block of exactly the bytes it needs, 2 MiB-aligned and then
// shifted by base_offset, so a lane that reads or writes past the end trips AddressSanitizer
// and a write before the start is caught by the sentinel bytes in front.
//
// SA_CASE_INCREMENT: the op adds 1 to i0 in place (out0 aliases in0), so "each vector is
//   visited exactly once" is the same as "each element ends at seed + 1".
// SA_CASE_MIXED: four arrays of different element widths; checks that narrow and wide arrays are
//   addressed with the same element index and that element_idx counts elements of the array.
// SA_CASE_NARROW: float in, short out: the input is the wider array, so ownership (striped or sided)
//   follows i0's address.
// SA_CASE_WIDEN: short in, float out: striped ownership follows o0, the sided map the narrower i0
//   (tiles of half as many bytes).
#include <cstdio>
#include <cstdlib>

#include "../../l2_torch_alloc_amd/csrc/launch_plan.h"

static unsigned g_stripe_log2 = 14, g_slot_run = 1, g_segments = 1;
// The word a launch planned with `dealing_from_memory` reads its dealing offset from (the driver
// sets it per case, to a value the plan does not know).
static unsigned int g_dealing_word = 0;
static bool g_dealing_from_memory = false;

// The plan for one array: the striped one, or, in an instantiation built with SA_SIDED, the sided
// one with an origin, arena constant and dealing offset derived from the case (any values must
// give a map that visits every tile once).
static sideaware::LaunchPlan make_plan(unsigned long long base, long long nv, unsigned grid) {
    if (sa_sided) {
        sideaware::SideMap side;
        side.origin_address = ((base * 2654435761ull) >> 7) & ~0x3fffull;
        side.pair_mask = SA_SIDE_PAIR_MASK;
        side.flip = (unsigned)(nv & 1);
        side.dealing = (unsigned)((grid + nv + g_stripe_log2) % SA_NUM_XCD);
        side.dealing_from_memory = g_dealing_from_memory;
        return sideaware::plan_launch_sided(base, nv, sideaware_kernel_meta[0], SA_NUM_XCD, g_stripe_log2 % 9,
                                            g_slot_run, grid / SA_NUM_XCD, side, (unsigned)sa_followed_vector_bytes);
    }
    return sideaware::plan_launch(base, nv, sideaware_kernel_meta[0], SA_NUM_XCD,
                                  1ull << g_stripe_log2, g_slot_run, grid / SA_NUM_XCD);
}

// `grid` is the caller's wish, as the launcher's parallel_groups would be: a persistent grid of
// that many workgroups (rounded to whole XCDs), or 0 for one workgroup per tile.  The plan is made
// by the same function the launcher uses.
static void run_grid(unsigned grid, size_type nv, vo0* o0, vo1* o1, vo2* o2, vo3* o3,
                     const vi0* i0, const vi1* i1, const vi2* i2, const vi3* i3, int* mem, int val) {
    if (g_segments > 1) {
        sa_batch_args batch;
        std::memset(&batch, 0, sizeof batch);
        batch.count = g_segments;
        unsigned blocks = 0;
        for (unsigned s = 0; s < g_segments; s++) {
            // cut points: increasing, rarely on a tile boundary, some pieces empty when nv is small
            auto cut = [&](unsigned i) -> long long {
                if (i == 0) return 0;
                if (i >= g_segments) return (long long)nv;
                const long long even = (long long)nv * i / g_segments, next = (long long)nv * (i + 1) / g_segments;
                const long long c = even + (i * 37) % 5;
                return c > next ? next : c;
            };
            const long long lo = cut(s), n = cut(s + 1) - lo;
            sa_segment_args& a = batch.segments.seg[s];
            a.output0 = o0 ? o0 + lo : nullptr; a.output1 = o1 ? o1 + lo : nullptr;
            a.output2 = o2 ? o2 + lo : nullptr; a.output3 = o3 ? o3 + lo : nullptr;
            a.input0 = i0 ? i0 + lo : nullptr; a.input1 = i1 ? i1 + lo : nullptr;
            a.input2 = i2 ? i2 + lo : nullptr; a.input3 = i3 ? i3 + lo : nullptr;
            a.mem = mem; a.val = val; a.num_vectors = n;
            const unsigned long long seg_base = sideaware_kernel_meta[2] ? (unsigned long long)a.output0
                                                                          : (unsigned long long)a.input0;
            sideaware::LaunchPlan p = make_plan(seg_base, n, grid);
            a.full_tiles = p.full_tiles; a.b0 = p.b0; a.u_count = p.u_count; a.run = p.run;
            a.r = p.r_word; a.tail_block = p.tail_block; a.first_block = blocks;
            blocks += p.grid;
            batch.blocks_end[s] = blocks;
        }
        for (unsigned s = g_segments; s < SA_MAX_SEGMENTS; s++) batch.blocks_end[s] = blocks;
        gridDim = {blocks, 1, 1};
        blockDim = {SA_WG_THREADS, 1, 1};
        for (unsigned b = 0; b < blocks; b++) {
            for (unsigned t = 0; t < SA_WG_THREADS; t++) {
                blockIdx = {b, 0, 0};
                threadIdx = {t, 0, 0};
                const unsigned* e = batch.blocks_end;
                SA_CONCAT(KERNEL_NAME, _batch)(batch.count, e[0], e[1], e[2], e[3], e[4], e[5], e[6], e[7],
                                               g_dealing_from_memory ? &g_dealing_word : nullptr, batch.segments);
            }
        }
        return;
    }
    const unsigned long long base = sideaware_kernel_meta[2] ? (unsigned long long)o0 : (unsigned long long)i0;
    sideaware::LaunchPlan p = make_plan(base, (long long)nv, grid);
    gridDim = {p.grid, 1, 1};
    blockDim = {SA_WG_THREADS, 1, 1};
    for (unsigned b = 0; b < p.grid; b++) {
        for (unsigned t = 0; t < SA_WG_THREADS; t++) {
            blockIdx = {b, 0, 0};
            threadIdx = {t, 0, 0};
            KERNEL_NAME(nv, (size_type)p.full_tiles, (size_type)p.b0, (size_type)p.u_count, (size_type)p.run,
                        p.r_word, p.grid, val, i0, o0, g_dealing_from_memory ? &g_dealing_word : nullptr, p.tail_block,
                        o1, o2, o3, i1, i2, i3, mem);
        }
    }
}

struct Arena {
    char* block = nullptr;
    char* data = nullptr;
    size_t off = 0;
    Arena(size_t offset, size_t bytes) : off(offset) {
        if (posix_memalign((void**)&block, 2u << 20, offset + bytes + (bytes == 0)) != 0) std::abort();
        std::memset(block, 0xAB, offset);
        data = block + offset;
    }
    bool sentinel_ok() const {
        for (size_t i = 0; i < off; i++) if ((unsigned char)block[i] != 0xAB) return false;
        return true;
    }
    ~Arena() { std::free(block); }
};

#if defined(SA_CASE_INCREMENT)
static int run_case(unsigned grid, long long nv, size_t off) {
    const size_t n = (size_t)nv * vec_size;
    Arena a(off, n * sizeof(int));
    int* x = (int*)a.data;
    for (size_t i = 0; i < n; i++) x[i] = (int)(i * 7u + 3u);
    run_grid(grid, (size_type)nv, (vo0*)x, nullptr, nullptr, nullptr, (const vi0*)x, nullptr, nullptr, nullptr,
             nullptr, 0);
    int bad = a.sentinel_ok() ? 0 : 1;
    for (size_t i = 0; i < n; i++) bad += (x[i] != (int)(i * 7u + 3u) + 1);
    return bad;
}
#elif defined(SA_CASE_MIXED)
static int run_case(unsigned grid, long long nv, size_t off) {
    const size_t n = (size_t)nv * vec_size;
    // only o0's array (the widest of i0/o0) is shifted by `off`; the narrower ones shift in proportion
    Arena f_out(off, n * sizeof(float)), s_out(off / 2, n * sizeof(short)), idx_out(off, n * sizeof(int));
    Arena s_in(off / 2, n * sizeof(short)), f_in(off, n * sizeof(float));
    short* si = (short*)s_in.data;
    float* fi = (float*)f_in.data;
    for (size_t i = 0; i < n; i++) { si[i] = (short)(i % 1000); fi[i] = (float)(i % 77) * 0.5f; }
    std::memset(f_out.data, 0, n * sizeof(float));
    std::memset(s_out.data, 0, n * sizeof(short));
    std::memset(idx_out.data, 0xff, n * sizeof(int));
    run_grid(grid, (size_type)nv, (vo0*)f_out.data, (vo1*)s_out.data, (vo2*)idx_out.data, nullptr,
             (const vi0*)si, (const vi1*)fi, nullptr, nullptr, nullptr, 5);
    int bad = 0;
    bad += !f_out.sentinel_ok() + !s_out.sentinel_ok() + !idx_out.sentinel_ok();
    for (size_t i = 0; i < n; i++) {
        bad += (((float*)f_out.data)[i] != (float)si[i] + fi[i]);
        bad += (((short*)s_out.data)[i] != (short)(fi[i] * 10.0f + 5.0f));
        bad += (((int*)idx_out.data)[i] != (int)i);
    }
    return bad;
}
#elif defined(SA_CASE_NARROW)
static int run_case(unsigned grid, long long nv, size_t off) {
    const size_t n = (size_t)nv * vec_size;
    // i0 is the wider array: it is the one shifted by `off` and the one the ownership map follows
    Arena f_in(off, n * sizeof(float)), s_out(off / 2, n * sizeof(short));
    float* fi = (float*)f_in.data;
    for (size_t i = 0; i < n; i++) fi[i] = (float)(i % 3001);
    std::memset(s_out.data, 0xff, n * sizeof(short));
    run_grid(grid, (size_type)nv, (vo0*)s_out.data, nullptr, nullptr, nullptr, (const vi0*)fi, nullptr, nullptr, nullptr,
             nullptr, 0);
    int bad = !s_out.sentinel_ok() + !f_in.sentinel_ok();
    for (size_t i = 0; i < n; i++) bad += (((short*)s_out.data)[i] != (short)(i % 3001) + 1);
    return bad;
}
#elif defined(SA_CASE_WIDEN)
static int run_case(unsigned grid, long long nv, size_t off) {
    const size_t n = (size_t)nv * vec_size;
    // o0 is the wider array (shifted by `off`); the only input is narrower, and a sided instantiation
    // follows it: half a tile of o0's bytes per tile
    Arena f_out(off, n * sizeof(float)), s_in(off / 2, n * sizeof(short));
    short* si = (short*)s_in.data;
    for (size_t i = 0; i < n; i++) si[i] = (short)(i % 3001);
    std::memset(f_out.data, 0xff, n * sizeof(float));
    run_grid(grid, (size_type)nv, (vo0*)f_out.data, nullptr, nullptr, nullptr, (const vi0*)si, nullptr, nullptr, nullptr,
             nullptr, 0);
    int bad = !f_out.sentinel_ok() + !s_in.sentinel_ok();
    for (size_t i = 0; i < n; i++) bad += (((float*)f_out.data)[i] != (float)(i % 3001) + 0.5f);
    return bad;
}
#elif defined(SA_CASE_ROPE)
// The op header under test is a generated RoPE header; rope_T / rope_half / rope_heads /
// rope_rotated come from it.  The activation holds `nv` vectors (any length: a whole number of
// tokens is not required, the decode must still stay inside the table), the table exactly
// rope_T * rope_half (cos, sin) pairs, so a wrong table index trips the sanitizer.  Expected
// values come from nested loops over (row, head, pair) that share no code with `indexing`.
static float rope_widen(float v) { return v; }
template<typename Tv> static float rope_widen(Tv v) { return (float)v; }
static int run_case(unsigned grid, long long nv, size_t off) {
    typedef decltype(i0().x) scalar;
    const size_t pairs = (size_t)nv * vec_size;
    Arena act(off, pairs * sizeof(i0));
    Arena table(0, (size_t)rope_T * rope_half * sizeof(float2));
    i0* x = (i0*)act.data;
    float2* f = (float2*)table.data;
    for (int t = 0; t < rope_T; t++)
        for (int d = 0; d < rope_half; d++) {
            f[(size_t)t * rope_half + d].x = (float)((t * 31 + d * 7) % 64) / 64.0f;
            f[(size_t)t * rope_half + d].y = (float)((t * 13 + d * 3) % 32) / 32.0f - 0.5f;
        }
    for (size_t p = 0; p < pairs; p++) {
        x[p].x = (scalar)((float)((p * 5) % 33) - 16.0f);
        x[p].y = (scalar)((float)((p * 11) % 17) - 8.0f);
    }
    i0* want = (i0*)std::malloc(pairs * sizeof(i0) + 1);
    for (size_t p = 0; p < pairs; p++) {
        size_t row = p / ((size_t)rope_heads * rope_half);      // (batch, token) flattened
        int head = (int)((p / rope_half) % rope_heads);
        int d = (int)(p % rope_half);
        int t = (int)(row % rope_T);
        want[p] = x[p];
        if (head < rope_rotated) {
            float re = rope_widen(x[p].x), im = rope_widen(x[p].y);
            float c = f[(size_t)t * rope_half + d].x, s = f[(size_t)t * rope_half + d].y;
            want[p].x = (scalar)(re * c - im * s);
            want[p].y = (scalar)(im * c + re * s);
        }
    }
    run_grid(grid, (size_type)nv, (vo0*)x, nullptr, nullptr, nullptr, (const vi0*)x, (const vi1*)f, nullptr, nullptr,
             nullptr, 0);
    int bad = act.sentinel_ok() ? 0 : 1;
    for (size_t p = 0; p < pairs; p++) bad += (std::memcmp(&x[p], &want[p], sizeof(i0)) != 0);
    std::free(want);
    return bad;
}
#else
#error "define SA_CASE_INCREMENT, SA_CASE_MIXED, SA_CASE_NARROW, SA_CASE_WIDEN or SA_CASE_ROPE"
#endif

int main() {
    unsigned grid;
    long long nv;
    size_t off;
    int cases = 0, failed = 0;
    char line[256];
    while (std::fgets(line, sizeof line, stdin)) {
        g_segments = 1;
        if (std::sscanf(line, "%u %lld %zu %u %u %u", &grid, &nv, &off, &g_stripe_log2, &g_slot_run, &g_segments) < 5) continue;
        if (g_segments < 1 || g_segments > SA_MAX_SEGMENTS) g_segments = 1;
        cases++;
        // every third case of a sided instantiation takes its dealing offset from memory
        g_dealing_from_memory = sa_sided && (cases % 3 == 0);
        g_dealing_word = 0x80000000u | (unsigned)((cases * 5 + nv) % SA_NUM_XCD);
        int bad = run_case(grid, nv, off);
        if (bad) {
            failed++;
            std::printf("FAIL grid=%u nv=%lld off=%zu stripe_log2=%u run=%u segments=%u: %d bad elements\n", grid, nv,
                        off, g_stripe_log2, g_slot_run, g_segments, bad);
        }
    }
    std::printf("cases=%d failed=%d\n", cases, failed);
    return failed ? 1 : 0;
}
