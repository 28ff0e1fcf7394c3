"""The sided ownership map on a real MI355X: what the library measures about the device's two
halves, which launches use the map, that results stay bit-exact whatever the host believes, and
that the workgroups really run on the half of the device that holds the bytes they touch.

The reference's counterpart is its L2-side machinery: the start-up side test and hash fit
(sideaware.cu:441-760), `sideaware_elementwise`'s side lookup (sideaware.cu:206-305) and the
FORCE_WRONG_SIDE switch (sideaware.cu:70-75)."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

MiB = 1 << 20
MI355X_SIDE_BITS = (1 << 13) | (1 << 21) | (1 << 28)

# One int per element: the id of the XCD the workgroup that wrote the element ran on.
XCD_ID_HEADER = b"""
#define KERNEL_NAME sideaware_test_xcd_id
typedef int o0;
typedef int i0;
struct unused {};
typedef unused o1, o2, o3, i1, i2, i3;
constexpr bool reverse_order = false;
constexpr bool input_evict[4] = {true, false, false, false};
__device__ __forceinline__ void elementwise_op(size_t element_idx, int sideband,
                                               o0 &out0, o1 &out1, o2 &out2, o3 &out3,
                                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {
    unsigned int xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    out0 = (int)(xcc & 0xf) + (in0 & 0);
}
"""

# A narrowing op (float in, short out): every output element is the id of the XCD its workgroup ran on.
NARROWING_XCD_ID_HEADER = b"""
#define KERNEL_NAME sideaware_test_narrowing_xcd_id
typedef short o0;
typedef float i0;
struct unused {};
typedef unused o1, o2, o3, i1, i2, i3;
constexpr bool reverse_order = false;
constexpr bool input_evict[4] = {true, false, false, false};
__device__ __forceinline__ void elementwise_op(size_t element_idx, int sideband,
                                               o0 &out0, o1 &out1, o2 &out2, o3 &out3,
                                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {
    unsigned int xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    out0 = (short)((xcc & 0xf) + (in0 != 0.0f ? 100 : 0));
}
"""

ADD_ONE_HEADER = b"""
#define KERNEL_NAME sideaware_test_add_one
typedef unsigned char o0;
typedef unsigned char i0;
struct unused {};
typedef unused o1, o2, o3, i1, i2, i3;
constexpr bool reverse_order = false;
constexpr bool input_evict[4] = {true, false, false, false};
__device__ __forceinline__ void elementwise_op(size_t element_idx, int sideband,
                                               o0 &out0, o1 &out1, o2 &out2, o3 &out3,
                                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {
    out0 = (unsigned char)(in0 + 1);
}
"""


def counts(lib):
    a, b = ctypes.c_ulonglong(), ctypes.c_ulonglong()
    lib.sideaware_launch_counts(ctypes.byref(a), ctypes.byref(b))
    return a.value, b.value


@pytest.fixture
def lib(sa):
    L = sa.library()
    if L.sideaware_side_address_mask() == 0:
        # the first large region makes the library measure the device
        torch.empty(64 * MiB, dtype=torch.uint8, device="cuda")
    if L.sideaware_side_address_mask() == 0:
        pytest.skip("the device showed no side structure to the start-up probe")
    yield L
    for key, value in ((b"sided", 1), (b"sided_wrong", 0), (b"sided_stripe", -1), (b"sided_min_bytes", 8 * MiB),
                       (b"sided_widening", 0), (b"sided_align", 16), (b"sided_agreement", 70)):
        assert L.sideaware_tune(key, value) == 0


def test_the_probe_finds_the_mi355x_side_hash(lib):
    assert lib.sideaware_side_address_mask() == MI355X_SIDE_BITS
    assert lib.sideaware_num_xcds() == 8


def test_side_of_follows_the_hash_and_large_regions_are_canonical(lib):
    t = torch.empty(96 * MiB, dtype=torch.uint8, device="cuda")
    p = t.data_ptr()
    # canonical placement: the region starts on side 0 and its sides follow parity(offset & bits)
    agree = 0
    offsets = [i * 8192 * 37 for i in range(300)]
    for o in offsets:
        agree += lib.sideaware_side_of(p + o) == bin(o & MI355X_SIDE_BITS).count("1") & 1
    assert agree >= 0.93 * len(offsets)
    assert lib.sideaware_side_of(p) == 0 and lib.sideaware_side_of(p + 8192) == 1
    assert lib.sideaware_side_of(p + 4096) == lib.sideaware_side_of(p)       # one granule is 8 KiB
    # memory the pool did not hand out has no known side
    assert lib.sideaware_side_of(ctypes.c_void_p(0x1000)) == -1


def test_which_launches_are_sided(sa, lib):
    stream = torch.cuda.current_stream().cuda_stream
    n = 64 * MiB
    src = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda")
    dst = torch.zeros_like(src)

    def copy(d, s, nbytes):
        before = counts(lib)
        lib.sideaware_memcpy(d, s, nbytes, 0, stream)
        torch.cuda.synchronize()
        after = counts(lib)
        return after[0] - before[0], after[1] - before[1]

    assert copy(dst.data_ptr(), src.data_ptr(), n) == (1, 0)                 # two canonical regions: sided
    assert torch.equal(dst, src)
    assert copy(dst.data_ptr(), src.data_ptr(), 4 * MiB) == (0, 1)           # too short to matter
    assert copy(dst.data_ptr() + 4096, src.data_ptr() + 4096, n - 8192) == (1, 0)      # not on a granule boundary: still sided
    assert copy(dst.data_ptr() + 1024 + 16, src.data_ptr() + 1024 + 16, n - 8192) == (1, 0)
    assert lib.sideaware_tune(b"sided_align", 8192) == 0                               # unless an alignment is demanded
    assert copy(dst.data_ptr() + 4096, src.data_ptr() + 4096, n - 8192) == (0, 1)
    assert lib.sideaware_tune(b"sided_align", 16) == 0
    assert torch.equal(dst, src)
    # the source's sides are the opposite of the destination's over the whole array: the launch
    # follows its source (loads stay on their own half, every store crosses: still faster than stripes)
    assert copy(dst.data_ptr(), src.data_ptr() + 2 * MiB, n - 2 * MiB) == (1, 0)
    assert torch.equal(dst[: n - 2 * MiB], src[2 * MiB:])
    # ... wherever the destination lies: only the source has to be in measured memory
    dst.zero_()
    assert copy(dst.data_ptr() + 4096 + 16, src.data_ptr(), n - 8192) == (1, 0)
    assert torch.equal(dst[4096 + 16: 4096 + 16 + n - 8192], src[: n - 8192])
    assert copy(dst.data_ptr(), src.data_ptr(), n) == (1, 0)
    assert lib.sideaware_tune(b"sided", 0) == 0
    assert copy(dst.data_ptr(), src.data_ptr(), n) == (0, 1)
    assert lib.sideaware_tune(b"sided", 1) == 0
    assert torch.equal(dst, src)
    # in place: the input is the output
    assert copy(dst.data_ptr(), dst.data_ptr(), n) == (1, 0)
    assert torch.equal(dst, src)
    # an op whose only input is narrower than its output is faster on the striped map; one with no
    # input at all follows its output
    widen = sa.sideaware_create_kernel(b"""
typedef float o0;
typedef __bf16 i0;
struct unused {};
typedef unused o1, o2, o3, i1, i2, i3;
constexpr bool reverse_order = false;
constexpr bool input_evict[4] = {true, false, false, false};
__device__ __forceinline__ void elementwise_op(size_t element_idx, int sideband, o0 &out0, o1 &out1, o2 &out2, o3 &out3,
                                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) { out0 = (float)in0; }
""")
    x = torch.randn(16 * MiB, device="cuda").to(torch.bfloat16)
    y = torch.empty(16 * MiB, device="cuda")
    before = counts(lib)
    lib.sideaware_one_to_one(widen, y.numel() * 4, y.data_ptr(), x.data_ptr(), 0, stream)
    torch.cuda.synchronize()
    assert counts(lib) == (before[0], before[1] + 1) and torch.equal(y, x.float())
    from l2_torch_alloc_amd import ops
    z = torch.empty(16 * MiB, dtype=torch.int32, device="cuda")
    before = counts(lib)
    ops.fill_int32(z, 7)
    torch.cuda.synchronize()
    assert counts(lib) == (before[0] + 1, before[1]) and bool((z == 7).all())
    # an op with no output at all (a scan that reports through the sideband pointer) follows its input
    scan = sa.sideaware_create_kernel(b"""
#define KERNEL_NAME sideaware_test_scan
typedef int i0;
struct unused {};
typedef unused o0, o1, o2, o3, i1, i2, i3;
constexpr bool reverse_order = false;
constexpr bool input_evict[4] = {true, false, false, false};
__device__ __forceinline__ void elementwise_op(size_t element_idx, int sideband, o0 &out0, o1 &out1, o2 &out2, o3 &out3,
                                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {}
#define CUSTOM_VECTOR_OP
__device__ __forceinline__ void vector_op(size_type vec_idx, int vec_size, o0 *out0, o1 *out1, o2 *out2, o3 *out3,
                                          const i0 *in0, const i1 *in1, const i2 *in2, const i3 *in3,
                                          int* sideband_memory, int sideband_value) {
    for (int i = 0; i < 4; i++) if (in0[i] == sideband_value) atomicAdd(sideband_memory, 1);
}
""")
    hits = torch.zeros(4, dtype=torch.int32, device="cuda")
    z[12345] = 8
    z[-1] = 8
    before = counts(lib)
    lib.sideaware_elementwise(scan, z.numel() * 4, 0, 0, 0, 0, z.data_ptr(), 0, 0, 0, hits.data_ptr(), 8, 0, 0, 0, stream)
    torch.cuda.synchronize()
    assert counts(lib) == (before[0] + 1, before[1]) and int(hits[0]) == 2
    # an op whose output is narrower than its input follows the input: the input must be in measured
    # memory, the output may be anywhere
    narrow = sa.sideaware_create_kernel(NARROWING_XCD_ID_HEADER)
    w = torch.zeros(16 * MiB, device="cuda")
    h = torch.empty(16 * MiB + 8, dtype=torch.int16, device="cuda")
    before = counts(lib)
    lib.sideaware_one_to_one(narrow, w.numel() * 4, h.data_ptr() + 16, w.data_ptr(), 0, stream)
    torch.cuda.synchronize()
    assert counts(lib) == (before[0] + 1, before[1])
    before = counts(lib)
    lib.sideaware_one_to_one(narrow, w.numel() * 4 - 8192, h.data_ptr(), w.data_ptr() + 4096, 0, stream)
    torch.cuda.synchronize()
    assert counts(lib) == (before[0] + 1, before[1])


def agreeing_offset(lib, base, nbytes, first):
    """The lowest multiple of 4 MiB at or above `first` such that [base + offset + 16 KiB, ...) has
    the same side as [base, ...) at (nearly) every offset."""
    a = (first + 4 * MiB - 1) // (4 * MiB) * (4 * MiB)
    samples = [(nbytes // 64) * i & ~0x1fff for i in range(64)]
    for _ in range(200):
        agree = sum(lib.sideaware_side_of(base + o) == lib.sideaware_side_of(base + a + 16384 + o) for o in samples)
        if agree >= 62:
            return a
        a += 4 * MiB
    raise AssertionError("no offset with matching sides found")


@pytest.mark.parametrize("nbytes", [8 * MiB, 8 * MiB + 16, 37 * MiB + 4096 + 48, 256 * MiB, 300 * MiB - 16])
def test_sided_copy_is_bit_exact_whatever_the_host_believes(sa, lib, nbytes):
    """Any arena constant, stripe and dealing offset gives a map that visits every vector once:
    wrong beliefs cost speed only."""
    stream = torch.cuda.current_stream().cuda_stream
    # source and destination are cut from one region, the destination where its sides match the
    # source's and with guard bytes on both ends
    big = torch.empty(2 * nbytes + 600 * MiB, dtype=torch.uint8, device="cuda")
    gen = torch.Generator(device="cuda").manual_seed(nbytes % 1000)
    src = big[:nbytes]
    src.copy_(torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device="cuda", generator=gen))
    at = agreeing_offset(lib, big.data_ptr(), nbytes, nbytes)
    assert at + 16384 + nbytes + 16384 <= big.numel()
    dst_all = big[at: at + 16384 + nbytes + 16384]
    dst = dst_all[16384: 16384 + nbytes]
    for wrong in (0, 1):
        for stripe in (-1, 0, 3, 7, 12):
            assert lib.sideaware_tune(b"sided_wrong", wrong) == 0 and lib.sideaware_tune(b"sided_stripe", stripe) == 0
            dst_all.fill_(0xA5)
            before = counts(lib)
            lib.sideaware_memcpy(dst.data_ptr(), src.data_ptr(), nbytes, 0, stream)
            torch.cuda.synchronize()
            assert counts(lib)[0] == before[0] + 1, "the launch was expected to use the sided map"
            assert torch.equal(dst, src), (wrong, stripe)
            assert bool((dst_all[:16384] == 0xA5).all()) and bool((dst_all[16384 + nbytes:] == 0xA5).all())
    assert sa.sideaware_last_error() == ""


def test_sided_copies_at_random_offsets_are_bit_exact(sa, lib):
    """Seeded random lengths, source offsets (on and off granule boundaries) and destination
    offsets (any multiple of 16 bytes: aligned and split-line stores, matching and opposite side
    patterns): every launch is sided, every byte arrives, none beside the destination changes."""
    import random
    stream = torch.cuda.current_stream().cuda_stream
    rng = random.Random(20)
    big_src = torch.randint(0, 256, (100 * MiB,), dtype=torch.uint8, device="cuda")
    big_dst = torch.empty(100 * MiB, dtype=torch.uint8, device="cuda")
    sided = 0
    for case in range(24):
        n = rng.randrange(8 * MiB, 96 * MiB) // 16 * 16
        s_off = rng.randrange(0, 2 * MiB // 8192) * 8192 + rng.choice([0, 0, 16, 64, 1024, 4096, 4096 + 48])
        d_off = rng.choice([0, 16, 64, 4096, 8192, 2 * MiB]) + rng.randrange(0, 4096 // 16) * 16 * rng.choice([0, 1])
        d_off = max(d_off, 64)                     # room for guard bytes in front
        big_dst.fill_(0xA5)
        before = counts(lib)
        lib.sideaware_memcpy(big_dst.data_ptr() + d_off, big_src.data_ptr() + s_off, n, 0, stream)
        torch.cuda.synchronize()
        sided += counts(lib)[0] - before[0]
        assert torch.equal(big_dst[d_off: d_off + n], big_src[s_off: s_off + n]), (case, n, s_off, d_off)
        assert bool((big_dst[d_off - 64: d_off] == 0xA5).all()) and bool((big_dst[d_off + n: d_off + n + 4096] == 0xA5).all()), (case, n, s_off, d_off)
    assert sided == 24
    assert not sa.sideaware_last_error()


@pytest.mark.parametrize("n", [16 * MiB, 64 * MiB, 256 * MiB, 1024 * MiB])
def test_every_workgroup_runs_on_the_side_of_its_bytes(sa, lib, n):
    """An op that stores the id of the XCD it runs on: after the stream's dealing offset has been
    fed back (one launch), every 8 KiB granule was handled by the half of the device that
    sideaware_side_of names for that granule of the source (the array a launch follows), and with the
    wrong-side switch by the other: what the queries report predicts where the work runs, in every
    size class of the launch planner (16 MiB, 64 MiB, 256 MiB, 1 GiB)."""
    stream = torch.cuda.current_stream().cuda_stream
    kid = sa.sideaware_create_kernel(XCD_ID_HEADER)
    src = torch.zeros(n // 4, dtype=torch.int32, device="cuda")
    out = torch.full((n // 4,), -1, dtype=torch.int32, device="cuda")
    for wrong in (0, 1):
        assert lib.sideaware_tune(b"sided_wrong", wrong) == 0
        for _ in range(3):                        # the first launch may still plan with a stale dealing offset
            before = counts(lib)
            lib.sideaware_one_to_one(kid, n, out.data_ptr(), src.data_ptr(), 0, stream)
            torch.cuda.synchronize()
            assert counts(lib)[0] == before[0] + 1
        xcd = out.view(-1, 8192 // 4)             # one row per granule
        assert bool((xcd == xcd[:, :1]).all()), "a granule was written from more than one XCD"
        assert int(xcd.min()) >= 0 and int(xcd.max()) <= 7
        half = (xcd[:, 0] // 4).cpu().tolist()
        step = 97 if n <= 64 * MiB else 997
        checked = 0
        for g in range(0, len(half), step):
            side = lib.sideaware_side_of(src.data_ptr() + g * 8192)
            assert side in (0, 1)
            assert half[g] == side ^ wrong, (g, half[g], side, wrong)
            checked += 1
        assert checked > 20
        # and the XCDs of a side share the work evenly
        per_xcd = torch.bincount(xcd[:, 0].flatten().cpu(), minlength=8).tolist()
        assert max(per_xcd) - min(per_xcd) <= len(half) // 64, per_xcd
    assert 0 <= lib.sideaware_stream_dealing(stream) <= 7


def test_sided_launches_replay_from_a_hip_graph(sa, lib):
    """The workgroups of a replayed graph node are dealt to the XCDs from another offset than
    those of a direct launch, and a captured launch's plan is frozen.  So a sided launch under
    stream capture is preceded (once per capture and stream) by a one-wave kernel that writes the
    XCD it runs on to a device word, and the launch's own kernel reads its dealing offset from
    that word at every replay.  Replays are bit-exact on the capture stream, on the default stream and on a third one, also with
    eager, sided work of the program's own between them, and the XCDs of a replayed launch sit on
    the side of the bytes they handle."""
    n = 64 * MiB
    src = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda")
    mid = torch.zeros_like(src)
    dst = torch.zeros_like(src)
    kid = sa.sideaware_create_kernel(XCD_ID_HEADER)
    zeros = torch.zeros(n // 4, dtype=torch.int32, device="cuda")
    where = torch.full((n // 4,), -1, dtype=torch.int32, device="cuda")
    torch.ops.sideaware.memcpy(mid, src)            # compiles outside the capture
    lib.sideaware_one_to_one(kid, n, where.data_ptr(), zeros.data_ptr(), 0, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    before = counts(lib)
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            torch.ops.sideaware.memcpy(mid, src)
            torch.ops.sideaware.memcpy(dst, mid)
            lib.sideaware_one_to_one(kid, n, where.data_ptr(), zeros.data_ptr(), 0, side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    assert counts(lib) == (before[0] + 3, before[1]), "the captured launches were not sided"
    sides = torch.tensor([lib.sideaware_side_of(zeros.data_ptr() + g * 8192) for g in range(0, n // 8192, 61)], device="cuda")
    other = torch.zeros(16 * MiB, dtype=torch.uint8, device="cuda")
    third = torch.cuda.Stream()
    for trial, replay_on in enumerate([torch.cuda.current_stream(), side, third, torch.cuda.current_stream()]):
        src.random_(0, 256)
        dst.zero_()
        where.fill_(-1)
        torch.ops.sideaware.memcpy(other, src[: 16 * MiB])      # eager work of the program's own between replays
        torch.cuda.synchronize()
        with torch.cuda.stream(replay_on):
            graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(dst, src), trial
        assert torch.equal(other, src[: 16 * MiB]), trial
        xcd = where.view(-1, 2048)
        assert bool((xcd == xcd[:, :1]).all()) and int(xcd.min()) >= 0 and int(xcd.max()) <= 7, trial
        wrong = int(((xcd[::61, 0] // 4) != sides).sum())
        assert wrong == 0, (trial, wrong)
    assert not sa.sideaware_last_error()


def test_a_sided_batch_replays_from_a_hip_graph(sa, lib):
    """q and k of a grouped-query model rotated in one batched launch (both long enough to be
    sided), captured into a graph: the replays give what the direct launch gives, bit for bit."""
    from l2_torch_alloc_amd import ops
    T, D = 4096, 128
    freqs = ops.freqs_cis_table(D, T, 500000.0).cuda()
    g = torch.Generator().manual_seed(5)
    q0 = torch.randn(1, T, 32, D, generator=g).to(torch.bfloat16).cuda()      # 32 MiB
    k0 = torch.randn(1, T, 8, D, generator=g).to(torch.bfloat16).cuda()       # 8 MiB
    want_q, want_k = q0.clone(), k0.clone()
    before = counts(lib)
    ops.rope_forward_heads_many([want_q, want_k], freqs)                       # direct, and compiles outside the capture
    torch.cuda.synchronize()
    assert counts(lib) == (before[0] + 1, before[1])
    q, k = q0.clone(), k0.clone()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    before = counts(lib)
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            ops.rope_forward_heads_many([q, k], freqs)
    torch.cuda.current_stream().wait_stream(side)
    assert counts(lib) == (before[0] + 1, before[1])
    for trial in range(3):
        q.copy_(q0)
        k.copy_(k0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(q, want_q) and torch.equal(k, want_k), trial
    assert not sa.sideaware_last_error()


def test_the_dealing_offset_survives_other_kernels_on_the_stream(sa, lib):
    """The sided map plans with the XCD that workgroup 0 of the stream's last sided launch ran on.
    That offset belongs to the queue, not to its history: kernels of other shapes in between (PyTorch's
    own, with odd workgroup counts) do not move it, so no sided launch after the first is planned
    with a stale offset."""
    import random
    stream = torch.cuda.current_stream().cuda_stream
    kid = sa.sideaware_create_kernel(XCD_ID_HEADER)
    n = 32 * MiB
    src = torch.zeros(n // 4, dtype=torch.int32, device="cuda")
    out = torch.full((n // 4,), -1, dtype=torch.int32, device="cuda")
    sides = torch.tensor([lib.sideaware_side_of(src.data_ptr() + g * 8192) for g in range(0, n // 8192, 61)], device="cuda")
    assert int(sides.min()) >= 0

    def launch():
        out.fill_(-1)
        believed = lib.sideaware_stream_dealing(stream)
        lib.sideaware_one_to_one(kid, n, out.data_ptr(), src.data_ptr(), 0, stream)
        torch.cuda.synchronize()
        wrong = int(((out.view(-1, 2048)[::61, 0] // 4) != sides).sum())
        return believed, lib.sideaware_stream_dealing(stream), wrong

    for _ in range(2):
        launch()
    rng = random.Random(1)
    for trial in range(12):
        for _ in range(rng.randrange(1, 5)):
            m = rng.choice([1, 3, 7, 100, 257, 4099, 65537]) * rng.choice([1, 64, 256])
            a = torch.empty(m, device="cuda").normal_()
            (a * 2 + 1).sum()
        believed, reported, wrong = launch()
        assert believed == reported and wrong == 0, (trial, believed, reported, wrong)


def test_a_stream_whose_offset_keeps_changing_goes_striped_until_it_settles(sa, lib):
    """The host plans a sided launch with the offset the stream's last sided launch reported.  A
    stream that reports another offset at every launch (forced here by overwriting the report, as a
    stream moved between hardware queues would) makes every plan wrong, so after a few changes its
    launches use the striped map, and go back to the sided one once the reports agree again.
    Results are exact throughout."""
    side = torch.cuda.Stream()
    stream = side.cuda_stream
    n = 32 * MiB
    src = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda")
    dst = torch.zeros_like(src)
    torch.cuda.synchronize()

    def launch():
        before = counts(lib)
        lib.sideaware_memcpy(dst.data_ptr(), src.data_ptr(), n, 0, stream)
        side.synchronize()
        after = counts(lib)
        return after[0] - before[0]

    assert [launch() for _ in range(4)] == [1, 1, 1, 1]
    true_offset = lib.sideaware_stream_dealing(stream)
    used = []
    for i in range(12):
        lib.sideaware_set_stream_dealing(stream, (true_offset + 1 + i % 3) % 8)     # never what the launch will report
        used.append(launch())
    assert used[:3] == [1, 1, 1] and 0 in used[3:], used
    assert sum(used[4:]) <= 3, used                      # mostly striped once the changes were noticed
    settled = [launch() for _ in range(24)]
    assert settled[-4:] == [1, 1, 1, 1], settled
    assert lib.sideaware_stream_dealing(stream) == true_offset
    assert torch.equal(dst, src)


def test_a_narrowing_op_runs_on_the_side_of_its_input(sa, lib):
    """float in, short out: the sided map follows the input (the wider array, two thirds of the
    traffic).  Every 8 KiB granule of the input is read, and its 4 KiB of output written, by an XCD
    of the half of the device that holds that input granule."""
    stream = torch.cuda.current_stream().cuda_stream
    kid = sa.sideaware_create_kernel(NARROWING_XCD_ID_HEADER)
    n = 16 * MiB                                   # elements: 64 MiB in, 32 MiB out
    src = torch.zeros(n, dtype=torch.float32, device="cuda")
    out = torch.full((n,), -1, dtype=torch.int16, device="cuda")
    for _ in range(3):                             # the first launch may still plan with a stale dealing offset
        before = counts(lib)
        lib.sideaware_one_to_one(kid, n * 4, out.data_ptr(), src.data_ptr(), 0, stream)
        torch.cuda.synchronize()
        assert counts(lib)[0] == before[0] + 1
    xcd = out.view(-1, 8192 // 4)                  # one row per input granule (2048 elements)
    assert bool((xcd == xcd[:, :1]).all()), "an input granule was handled by more than one XCD"
    assert int(xcd.min()) >= 0 and int(xcd.max()) <= 7
    half = (xcd[:, 0] // 4).cpu().tolist()
    checked = 0
    for g in range(0, len(half), 97):
        side = lib.sideaware_side_of(src.data_ptr() + g * 8192)
        assert side in (0, 1)
        assert half[g] == side, (g, half[g], side)
        checked += 1
    assert checked > 50
    assert not sa.sideaware_last_error()


def test_a_batch_of_narrowing_segments_is_sided_segment_by_segment(sa, lib):
    """Several arrays in one launch of a narrowing op: every segment follows its own input (its
    own arena constants and origin), so in each of them an input granule is handled by one XCD of
    the half of the device that holds it."""
    from l2_torch_alloc_amd import ops
    kid = sa.sideaware_create_kernel(NARROWING_XCD_ID_HEADER)
    sizes = [12 * MiB, 8 * MiB + 2048, 20 * MiB]              # elements; the middle one ends in a partial tile
    srcs = [torch.zeros(n, dtype=torch.float32, device="cuda") for n in sizes]
    outs = [torch.full((n,), -1, dtype=torch.int16, device="cuda") for n in sizes]
    segments = [(n * 4, [o], [x], None, 0) for n, o, x in zip(sizes, outs, srcs)]
    for _ in range(3):
        before = counts(lib)
        ops.elementwise_batch(kid, segments)
        torch.cuda.synchronize()
        assert counts(lib) == (before[0] + 1, before[1])
    for n, o, x in zip(sizes, outs, srcs):
        assert int(o.min()) >= 0 and int(o.max()) <= 7
        whole = n // 2048 * 2048
        xcd = o[:whole].view(-1, 2048)                         # one row per input granule
        assert bool((xcd == xcd[:, :1]).all())
        half = (xcd[:, 0] // 4).cpu().tolist()
        for g in range(0, len(half), 53):
            assert half[g] == lib.sideaware_side_of(x.data_ptr() + g * 8192), (n, g)
    assert not sa.sideaware_last_error()


def test_a_widening_op_is_striped_unless_asked_and_then_follows_its_input(sa, lib):
    """short in, int out (every input narrower than the output): striped by default, which is as
    fast for such ops; with the `sided_widening` switch the sided map follows the input, so each
    8 KiB input granule and the 16 KiB of output it becomes are handled by one XCD of the half of
    the device that holds the input granule."""
    stream = torch.cuda.current_stream().cuda_stream
    kid = sa.sideaware_create_kernel(b"""
#define KERNEL_NAME sideaware_test_widening_xcd_id
typedef int o0;
typedef short i0;
struct unused {};
typedef unused o1, o2, o3, i1, i2, i3;
constexpr bool reverse_order = false;
constexpr bool input_evict[4] = {true, false, false, false};
__device__ __forceinline__ void elementwise_op(size_t element_idx, int sideband,
                                               o0 &out0, o1 &out1, o2 &out2, o3 &out3,
                                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {
    unsigned int xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    out0 = (int)(xcc & 0xf) + 1000 * (int)in0;
}
""")
    n = 16 * MiB                                   # elements: 32 MiB in, 64 MiB out
    src = torch.randint(0, 100, (n,), dtype=torch.int16, device="cuda")
    out = torch.full((n,), -1, dtype=torch.int32, device="cuda")
    before = counts(lib)
    lib.sideaware_one_to_one(kid, n * 4, out.data_ptr(), src.data_ptr(), 0, stream)
    torch.cuda.synchronize()
    assert counts(lib) == (before[0], before[1] + 1)
    assert torch.equal(out // 1000, src.int())
    assert lib.sideaware_tune(b"sided_widening", 1) == 0
    try:
        for _ in range(3):                         # the first launch may still plan with a stale dealing offset
            out.fill_(-1)
            before = counts(lib)
            lib.sideaware_one_to_one(kid, n * 4, out.data_ptr(), src.data_ptr(), 0, stream)
            torch.cuda.synchronize()
            assert counts(lib) == (before[0] + 1, before[1])
    finally:
        assert lib.sideaware_tune(b"sided_widening", 0) == 0
    assert torch.equal(out // 1000, src.int())
    xcd = (out % 1000).view(-1, 8192 // 2)         # one row per input granule (4096 elements)
    assert bool((xcd == xcd[:, :1]).all()), "an input granule was handled by more than one XCD"
    half = (xcd[:, 0] // 4).cpu().tolist()
    checked = 0
    for g in range(0, len(half), 97):
        side = lib.sideaware_side_of(src.data_ptr() + g * 8192)
        assert side in (0, 1)
        assert half[g] == side, (g, half[g], side)
        checked += 1
    assert checked > 40
    assert not sa.sideaware_last_error()


def test_registered_foreign_memory_gets_sided_launches(sa, lib):
    """Memory straight from hipMalloc is unknown to the pool: launches over it are striped and
    sideaware_side_of says -1.  Once registered, its sides are measured like an arena's: side_of
    answers (and agrees with a fresh probe), an in-place launch over it is sided, and results stay
    bit-exact.  Unregistered, it is unknown again."""
    stream = torch.cuda.current_stream().cuda_stream
    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipMalloc.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t]
    hip.hipMalloc.restype = ctypes.c_int
    hip.hipFree.argtypes = [ctypes.c_void_p]
    hip.hipFree.restype = ctypes.c_int
    hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
    hip.hipMemcpy.restype = ctypes.c_int
    n = 256 * MiB
    raw = ctypes.c_void_p()
    assert hip.hipMalloc(ctypes.byref(raw), n) == 0 and raw.value
    try:
        base = raw.value
        assert base % 16384 == 0
        seed = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda")
        back = torch.empty_like(seed)
        assert hip.hipMemcpy(base, seed.data_ptr(), n, 3) == 0               # device to device
        kid = sa.sideaware_create_kernel(ADD_ONE_HEADER)

        def add_one_in_place():
            before = counts(lib)
            lib.sideaware_one_to_one(kid, n, base, base, 0, stream)
            torch.cuda.synchronize()
            after = counts(lib)
            return after[0] - before[0], after[1] - before[1]

        assert lib.sideaware_side_of(base) == -1
        assert add_one_in_place() == (0, 1)
        assert lib.sideaware_register_region(base + 4096, n - 4096, 0) == -1      # not on a 16 KiB boundary
        assert "16 KiB" in sa.sideaware_last_error()
        lib.sideaware_clear_error()
        known = lib.sideaware_register_region(base, n, 0)
        assert known in (0, 1)
        if known == 0:
            pytest.skip("this allocation's sides did not fit the hash (not one physically contiguous run)")
        assert lib.sideaware_register_region(base, n, 0) == 0                     # overlaps what is known
        assert lib.sideaware_side_of(base) in (0, 1)
        assert lib.sideaware_side_of(base) != lib.sideaware_side_of(base + 8192)
        count = 128
        sides = torch.full((count,), -2, dtype=torch.int32, device="cuda")
        assert lib.sideaware_probe_sides(base, n, 99, count, sides.data_ptr(), 0, stream) == 0
        torch.cuda.synchronize()
        granules = n // 8192
        disagree = 0
        for i, s_i in enumerate(sides.cpu().tolist()):
            g = splitmix64(99 + i) % granules
            if s_i >= 0:
                disagree += s_i != lib.sideaware_side_of(base + g * 8192)
        assert disagree <= count // 32
        assert add_one_in_place() == (1, 0)
        assert add_one_in_place() == (1, 0)
        lib.sideaware_unregister_region(base, 0)
        assert lib.sideaware_side_of(base) == -1
        assert add_one_in_place() == (0, 1)
        assert hip.hipMemcpy(back.data_ptr(), base, n, 3) == 0
        assert torch.equal(back, seed + 4)                                         # uint8 arithmetic wraps
    finally:
        lib.sideaware_unregister_region(raw, 0)
        torch.cuda.synchronize()
        assert hip.hipFree(raw) == 0
    assert not sa.sideaware_last_error()


def test_sided_elementwise_with_two_inputs_and_mixed_widths(sa, lib):
    """bf16 x -> fp32 y (the output is the wider array, so the map follows it) and a two-input
    fp32 op, both compared with torch."""
    header = b"""
typedef float o0;
typedef __bf16 i0;
typedef float i1;
struct unused {};
typedef unused o1, o2, o3, i2, i3;
constexpr bool reverse_order = false;
constexpr bool input_evict[4] = {true, true, false, false};
__device__ __forceinline__ void elementwise_op(size_t element_idx, int sideband,
                                               o0 &out0, o1 &out1, o2 &out2, o3 &out3,
                                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {
    out0 = (float)in0 * 2.0f + in1;
}
"""
    stream = torch.cuda.current_stream().cuda_stream
    kid = sa.sideaware_create_kernel(header)
    n = 12 * MiB + 1000 * 4                       # elements; the fp32 arrays are 48 MiB + a tail
    x = torch.randn(n, device="cuda").to(torch.bfloat16)
    b = torch.randn(n, device="cuda")
    y = torch.empty(n, device="cuda")
    before = counts(lib)
    lib.sideaware_elementwise(kid, n * 4, y.data_ptr(), 0, 0, 0, x.data_ptr(), b.data_ptr(), 0, 0, 0, 0, 0, 0, 0, stream)
    torch.cuda.synchronize()
    assert counts(lib)[0] == before[0] + 1
    assert torch.equal(y, x.float() * 2.0 + b)


M64 = (1 << 64) - 1


def splitmix64(x):
    z = (x * 0x9e3779b97f4a7c15 + 0x9e3779b97f4a7c15) & M64
    z = ((z ^ (z >> 30)) * 0xbf58476d1ce4e5b9) & M64
    z = ((z ^ (z >> 27)) * 0x94d049bb133111eb) & M64
    return z ^ (z >> 31)


def test_probe_sides_measures_what_the_arena_probe_measured(sa, lib):
    """sideaware_probe_sides times loads at seeded sample granules of any device memory; on the
    pool's own memory its answers must be those of sideaware_side_of (measured once, when the arena
    was acquired), wherever the timing was decisive."""
    stream = torch.cuda.current_stream().cuda_stream
    region = torch.empty(320 * MiB, dtype=torch.uint8, device="cuda")
    count, seed, nbytes = 300, 5, 320 * MiB
    sides = torch.full((count + 4,), 9, dtype=torch.int32, device="cuda")
    assert lib.sideaware_probe_sides(region.data_ptr(), nbytes, seed, count, sides.data_ptr(), 0, stream) == 0
    torch.cuda.synchronize()
    got = sides.cpu().tolist()
    assert got[count:] == [9] * 4
    decisive = differ = 0
    for i in range(count):
        offset = (splitmix64((seed + i) & M64) % (nbytes // 8192)) * 8192
        want = lib.sideaware_side_of(region.data_ptr() + offset)
        assert want in (0, 1) and got[i] in (-1, 0, 1)
        decisive += got[i] >= 0
        differ += got[i] >= 0 and got[i] != want
    # a timing can go wrong, and a stretch of an arena can lie elsewhere than the arena's own probe
    # concluded from its samples: a few in a hundred may differ, not more
    assert decisive >= 0.9 * count and differ <= 0.03 * count, (decisive, differ)
    # bad arguments are refused with a message, nothing is launched
    assert lib.sideaware_probe_sides(region.data_ptr(), 64 * MiB, 1, 8, sides.data_ptr(), 0, stream) != 0
    assert b"128 MiB" in lib.sideaware_last_error()
    assert lib.sideaware_probe_sides(region.data_ptr() + 16, nbytes - 8192, 1, 8, sides.data_ptr(), 0, stream) != 0
    assert lib.sideaware_probe_sides(region.data_ptr(), nbytes, 1, 0, sides.data_ptr(), 0, stream) != 0
    lib.sideaware_clear_error()
