"""sideaware_probe_sides_noalloc, the entry point that allocates nothing, against
sideaware_probe_sides (the same measurement with an allocated work space), through the C ABI."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

MiB = 1 << 20
M64 = (1 << 64) - 1


def splitmix64(x):
    z = (x * 0x9e3779b97f4a7c15 + 0x9e3779b97f4a7c15) & M64
    z = ((z ^ (z >> 30)) * 0xbf58476d1ce4e5b9) & M64
    z = ((z ^ (z >> 27)) * 0x94d049bb133111eb) & M64
    return z ^ (z >> 31)


def test_the_allocation_free_probe_gives_what_the_allocating_one_gives(sa):
    lib = sa.library()
    if lib.sideaware_side_address_mask() == 0:
        pytest.skip("the device showed no side structure to the start-up probe")
    stream = torch.cuda.current_stream().cuda_stream
    region = torch.empty(384 * MiB, dtype=torch.uint8, device="cuda")
    base = region.data_ptr()
    # two calls in a row, the second with fewer samples (the static work array keeps the first call's
    # contents: what must start at zero is cleared by the entry point itself)
    for count, nbytes, seed in ((400, 384 * MiB, 11), (96, 256 * MiB, 12)):
        print("probe: count %d, %d MiB, seed %d" % (count, nbytes // MiB, seed), flush=True)
        want = torch.full((count + 8,), 77, dtype=torch.int32, device="cuda")
        got = torch.full((count + 8,), 77, dtype=torch.int32, device="cuda")
        before = sa.sideaware_alloc_stats()
        free_before = torch.cuda.mem_get_info()[0]
        assert lib.sideaware_probe_sides_noalloc(base, nbytes, seed, count, got.data_ptr(), 0, stream) == 0
        assert torch.cuda.mem_get_info()[0] == free_before                    # nothing was taken from the driver
        assert sa.sideaware_alloc_stats() == before                           # nor from the pool
        assert lib.sideaware_probe_sides(base, nbytes, seed, count, want.data_ptr(), 0, stream) == 0
        torch.cuda.synchronize()
        assert sa.sideaware_last_error() == ""
        g, w = got.cpu().tolist(), want.cpu().tolist()
        assert g[count:] == [77] * 8 and w[count:] == [77] * 8               # nothing written past `count`
        g, w = g[:count], w[:count]
        assert set(g) <= {-1, 0, 1} and set(w) <= {-1, 0, 1}
        # the two entry points agree wherever both measurements were decisive, and nearly all are
        # (the output is a timing measurement: the same sample can, rarely, come out differently twice)
        both = [(a, b) for a, b in zip(g, w) if a >= 0 and b >= 0]
        assert len(both) >= 0.9 * count
        assert sum(a != b for a, b in both) <= 0.02 * count, [(i, a, b) for i, (a, b) in enumerate(zip(g, w)) if a != b]
        # and both say what the pool measured for this arena when it acquired it (a timing can go
        # wrong: a few samples in a hundred may differ, not more)
        differ = 0
        for i in range(count):
            offset = (splitmix64((seed + i) & M64) % (nbytes // 8192)) * 8192
            side = lib.sideaware_side_of(base + offset)
            assert side in (0, 1)
            differ += (g[i] >= 0 and g[i] != side) + (w[i] >= 0 and w[i] != side)
        assert differ <= 0.03 * 2 * count, differ
    # more samples than the static array holds, and a region too short to scrub the L2s with: refused
    out = torch.zeros(1024, dtype=torch.int32, device="cuda")
    assert lib.sideaware_probe_sides_noalloc(base, 384 * MiB, 1, 513, out.data_ptr(), 0, stream) != 0
    assert b"static work array holds 512" in lib.sideaware_last_error()
    lib.sideaware_clear_error()
    assert lib.sideaware_probe_sides_noalloc(base, 64 * MiB, 1, 16, out.data_ptr(), 0, stream) != 0
    lib.sideaware_clear_error()
    torch.cuda.synchronize()
    assert bool((out == 0).all())
