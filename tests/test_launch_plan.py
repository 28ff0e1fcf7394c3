"""The launch planner (l2_torch_alloc_amd/csrc/launch_plan.h) against a brute-force model of what
the kernel does with a plan: every tile of the array is claimed by exactly one (workgroup, loop
trip), the partial last tile by exactly one workgroup, for any base, length, stripe, run and grid.
The kernel template itself is exercised with the same planner in test_kernel_cpu.py; this test is
the cheap, wide one (thousands of cases in pure Python)."""
import ctypes
import random

import pytest

from test_pool import build_harness


@pytest.fixture(scope="module")
def plan():
    L = ctypes.CDLL(build_harness())
    L.ph_plan_launch.argtypes = [ctypes.c_uint64, ctypes.c_longlong, ctypes.c_int, ctypes.c_int, ctypes.c_uint64,
                                 ctypes.c_longlong, ctypes.c_longlong, ctypes.POINTER(ctypes.c_longlong)]

    def call(base, nv, tile, xcds, stripe, run, slots):
        out = (ctypes.c_longlong * 8)()
        L.ph_plan_launch(base, nv, tile, xcds, stripe, run, slots, out)
        return dict(zip(("full_tiles", "b0", "u_count", "run", "r", "tail_block", "slots", "grid"), out))
    return call


def tiles_claimed(p, xcds):
    """The kernel's loop (elementwise_kernel.hip.inc), per workgroup, in Python."""
    claimed = []
    for block in range(p["grid"]):
        xcd, slot = block % xcds, block // xcds
        u_lin, in_run = slot * p["run"], 0
        while u_lin < p["u_count"]:
            u = u_lin
            u_lin += 1
            in_run += 1
            if in_run == p["run"]:
                in_run = 0
                u_lin += (p["slots"] - 1) * p["run"]
            a = ((((u >> p["r"]) * xcds) + xcd) << p["r"]) + (u & ((1 << p["r"]) - 1))
            g = a - p["b0"]
            if 0 <= g < p["full_tiles"]:
                claimed.append(g)
    return claimed


def test_every_tile_exactly_once(plan):
    rng = random.Random(11)
    for _ in range(1500):
        xcds = rng.choice([1, 2, 8])
        tile = 256 * rng.choice([1, 2, 3, 4, 8])
        nv = rng.choice([0, 1, tile - 1, tile, tile + 1, rng.randrange(0, 300 * tile)])
        base = rng.choice([0, 16, 4096, 1 << 21, (1 << 21) + 4096 * 5 + 48, rng.randrange(0, 1 << 30) * 16])
        stripe = 1 << rng.randrange(12, 25)
        run = rng.choice([0, 1, 2, 7, 64])
        slots = rng.choice([0, 1, 3, 32, 256])
        p = plan(base, nv, tile, xcds, stripe, run, slots)
        assert p["grid"] == p["slots"] * xcds and p["slots"] >= 1 and p["run"] >= 1
        assert p["slots"] <= max(1, p["u_count"])
        assert p["full_tiles"] == nv // tile
        claimed = tiles_claimed(p, xcds)
        assert sorted(claimed) == list(range(p["full_tiles"])), (base, nv, tile, xcds, stripe, run, slots)
        if nv % tile:
            assert 0 <= p["tail_block"] < p["grid"]
        else:
            assert p["tail_block"] == -1


def test_owner_depends_on_the_address_not_on_the_array(plan):
    # two arrays whose bases differ by a whole number of stripe periods, or by a few tiles: a byte's
    # owner XCD is a function of its address
    xcds, tile, stripe = 8, 256, 1 << 14
    tile_bytes = tile * 16
    r = 2                                            # 16 KiB stripe = 4 tiles of 4 KiB

    def owner(base, g):
        p = plan(base, 1000 * tile, tile, xcds, stripe, 1, 32)
        assert p["r"] == r
        a = p["b0"] + g
        return (a >> r) % xcds

    for base_a, base_b in ((0, 8 * stripe), (1 << 21, 5 * (1 << 21)), (4096 * 3, 4096 * 3 + 8 * stripe)):
        assert [owner(base_a, g) for g in range(100)] == [owner(base_b, g) for g in range(100)]
    # shifted by 5 tiles: tile g of one array is tile g+5 of the other, same address, same owner
    assert [owner(0, g + 5) for g in range(100)] == [owner(5 * tile_bytes, g) for g in range(100)]


def test_one_workgroup_per_tile_mode(plan):
    p = plan(1 << 21, 65536 * 256, 256, 8, 1 << 14, 1, 0)       # 256 MiB, aligned
    assert p["grid"] == 65536 and p["slots"] == p["u_count"] == 8192 and p["run"] == 1
    p = plan(1 << 21, 16, 256, 8, 1 << 14, 1, 0)                # 256 bytes: one workgroup group, tail only
    assert p["full_tiles"] == 0 and p["grid"] == 8 and 0 <= p["tail_block"] < 8
