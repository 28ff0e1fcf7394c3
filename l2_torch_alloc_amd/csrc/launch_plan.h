// Host-side planning of one launch of the elementwise kernel: everything about the workgroup ->
// tile map that does not depend on the workgroup is computed once here and handed to the kernel
// as scalars, so a workgroup's prologue has no divisions in it.  Plain C++ (no HIP), shared by the
// launcher and by the CPU harness that runs the kernel template lane by lane.
//
// Vocabulary (the kernel template uses the same names):
//   vector      16 bytes of the widest of (i0, o0)
//   tile        tile_vectors consecutive vectors: what one workgroup handles per loop trip
//   stripe      2^r consecutive tiles; stripe k of the address space belongs to XCD k % num_xcds
//   a           tile number counted from the last stripe-period boundary at or below the base
//   g = a - b0  tile number counted from the start of the array
//   u           XCD-local tile number: the XCD's tiles in address order
//   slots       workgroups per XCD; workgroup (xcd, slot) takes runs of `run` consecutive u,
//               `slots` runs apart
#pragma once

#include <cstdint>

namespace sideaware {

struct LaunchPlan {
    long long num_vectors = 0;
    long long full_tiles = 0;   // whole tiles in the array
    long long b0 = 0;           // tiles between the period boundary and the array's base
    long long u_count = 0;      // XCD-local tile numbers to cover (some map outside the array)
    long long run = 1;
    unsigned int r = 0;         // log2(tiles per stripe)
    int tail_block = -1;        // blockIdx.x of the workgroup that handles the partial last tile
    unsigned int slots = 1;     // workgroups per XCD
    unsigned int grid = 0;      // slots * num_xcds
};

// base_address: address of the array that defines ownership (o0's if o0 is wider than i0, else i0's).
// slots_wanted: workgroups per XCD for a persistent launch; 0 asks for one workgroup per tile.
// slot_run:     tiles a workgroup takes in a row; 0 gives each workgroup one contiguous block.
inline LaunchPlan plan_launch(uint64_t base_address, long long num_vectors, int tile_vectors, int num_xcds,
                              uint64_t stripe_bytes, long long slot_run, long long slots_wanted) {
    LaunchPlan p;
    const uint64_t tile_bytes = (uint64_t)tile_vectors * 16;
    p.num_vectors = num_vectors;
    p.r = 0;
    while (p.r < 20 && (tile_bytes << (p.r + 1)) <= stripe_bytes) p.r++;
    const long long period = (long long)num_xcds << p.r;
    p.b0 = (long long)((base_address / tile_bytes) % (uint64_t)period);
    p.full_tiles = num_vectors / tile_vectors;
    const long long a_end = p.b0 + p.full_tiles;
    p.u_count = ((a_end + period - 1) / period) << p.r;

    long long slots = slots_wanted > 0 ? slots_wanted : p.u_count;
    if (slots > p.u_count) slots = p.u_count;      // workgroups beyond the tile count would idle
    if (slots < 1) slots = 1;
    p.slots = (unsigned int)slots;
    p.grid = p.slots * (unsigned int)num_xcds;

    // A run longer than a workgroup's whole share is the same as the share (and keeps
    // slots * run within twice u_count, so the kernel's 32-bit stepping cannot overflow).
    const long long share = (p.u_count + slots - 1) / slots;
    p.run = slot_run > 0 && slot_run < share ? slot_run : share;
    if (p.run < 1) p.run = 1;

    if (p.full_tiles * tile_vectors < num_vectors) {
        const long long a = p.b0 + p.full_tiles;
        const long long stripe = a >> p.r;
        const long long owner_xcd = stripe % num_xcds;
        const long long u = ((stripe / num_xcds) << p.r) + (a & (((long long)1 << p.r) - 1));
        const long long owner_slot = (u / p.run) % slots;
        p.tail_block = (int)(owner_slot * num_xcds + owner_xcd);
    }
    return p;
}

}  // namespace sideaware
