"""Experiment modes of bench.py: A/B runs behind the design choices, each meant to be run alone
(often under rocprofv3) and each printing one JSON object.  The summaries under profiles/ name the
command that made them.

    python bench.py --stripe-ab | --chain-policy | --inflight-ab | --cache-probe | --ceiling | --rope-shapes
"""
import ctypes
import os

from bench_util import GiB, HBM_PEAK_GBPS, MiB, _abi, gbps, log, time_region


def stripe_ab(steps):
    """A/B evidence for the stripe -> XCD map, meant to be run under `rocprofv3 --pmc FETCH_SIZE`:
    the q RoPE with 4 KiB tiles (half a token row), once with 4 KiB ownership stripes, so the two
    halves of a row go to two XCDs and both L2s fetch the row's table entries, and once with 16 KiB
    and 256 KiB stripes, where a row stays on one XCD.  Kernel names carry the stripe size."""
    import torch
    from l2_torch_alloc_amd import headers, ops, wrapper
    lib, stream = _abi()
    B, T, HS = 8, 4096, 128
    q = torch.randn(B, T, 32, HS, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16).cuda()
    freqs = ops.freqs_cis_table(HS, T, 500000.0).cuda()
    nbytes = q.numel() * 2
    out = {}
    for stripe in (4096, 16384, 262144):
        assert lib.sideaware_tune(b"stripe_bytes", stripe) == 0
        text = headers.rope_header(T, 32, 0, HS, "bf16", "heads", unrolled=1, stream_output=True).decode()
        text = text.replace("#define KERNEL_NAME ", "#define KERNEL_NAME stripe%d_" % stripe)
        kid = wrapper.sideaware_create_kernel(text.encode())
        sec = time_region(lambda: lib.sideaware_elementwise(kid, nbytes, q.data_ptr(), 0, 0, 0, q.data_ptr(),
                                                            freqs.data_ptr(), 0, 0, 0, 0, 0, 0, 0, stream), steps, 2)
        out["stripe_%d" % stripe] = {"us": sec * 1e6, "GBps": gbps(2 * nbytes + freqs.numel() * 4, sec)}
    assert lib.sideaware_tune(b"stripe_bytes", 0) == 0
    return out


def chain_policy(reps=6):
    """The evidence behind the cache-policy classes: a producer launch followed at once by a consumer
    that reads its result (this library's copy), over buffer sets that cycle so that nothing is
    cache-resident, with the producer's stores left cacheable ("plain": OUTPUT_STREAMING 0) or
    streaming ("nt": OUTPUT_STREAMING 1).  Producers: a copy (not in
    place) and the bf16 RoPE (in place), at several sizes.  Per-launch times from HIP events."""
    import torch
    from l2_torch_alloc_amd import headers, ops, wrapper
    lib, stream = _abi()
    T, HS = 4096, 128
    freqs = ops.freqs_cis_table(HS, T, 500000.0).cuda()
    copy_text = headers.memcpy_header().decode()

    def producer_kernel(kind, stream_out, heads=32):
        tag = "chain_%s_%s_" % (kind, "nt" if stream_out else "plain")
        if kind == "copy":
            text = "#define INPUT0_STREAMING 1\n#define OUTPUT_STREAMING %d\n" % stream_out + copy_text
        else:
            text = headers.rope_header(T, heads, 0, HS, "bf16", "heads", stream_input=True,
                                       stream_output=bool(stream_out)).decode()
        return wrapper.sideaware_create_kernel(text.replace("#define KERNEL_NAME ", "#define KERNEL_NAME " + tag).encode())

    def run(kind, nbytes, stream_out, heads=32):
        kid = producer_kernel(kind, stream_out, heads)
        sets = min(24, max(3, (1536 * MiB) // (2 * nbytes)))
        srcs = [torch.randn(nbytes // 2, device="cuda").to(torch.bfloat16) for _ in range(sets)]
        mids = srcs if kind == "rope" else [torch.empty_like(t) for t in srcs]
        outs = [torch.empty_like(t) for t in srcs]
        evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(sets)]
        tp = tc = 0.0
        for rep in range(reps + 1):
            for i in range(sets):
                e = evs[i]
                e[0].record()
                lib.sideaware_elementwise(kid, nbytes, mids[i].data_ptr(), 0, 0, 0, srcs[i].data_ptr(),
                                          freqs.data_ptr() if kind == "rope" else 0, 0, 0, 0, 0, 0, 0, 0, stream)
                e[1].record()
                lib.sideaware_memcpy(outs[i].data_ptr(), mids[i].data_ptr(), nbytes, 0, stream)
                e[2].record()
            torch.cuda.synchronize()
            if rep:                                   # the first pass warms up
                tp += sum(e[0].elapsed_time(e[1]) for e in evs)
                tc += sum(e[1].elapsed_time(e[2]) for e in evs)
        n = reps * sets
        return {"producer_us": tp / n * 1e3, "consumer_us": tc / n * 1e3, "total_us": (tp + tc) / n * 1e3, "sets": sets}

    out = {}
    for mib in (32, 64, 128, 256):
        for stream_out in (0, 1):
            out["copy_%dMiB_stores_%s" % (mib, "nt" if stream_out else "plain")] = run("copy", mib * MiB, stream_out)
    for batch in (1, 2, 4, 8):                        # (batch, 4096, 32, 128) bf16 = batch * 32 MiB
        for stream_out in (0, 1):
            out["rope_in_place_%dMiB_stores_%s" % (batch * 32, "nt" if stream_out else "plain")] = \
                run("rope", batch * 32 * MiB, stream_out)
    return out


READ_ONLY_HEADER = """
#define KERNEL_NAME sideaware_read_only_%s
#define INPUT0_STREAMING %d
typedef int i0;
struct unused {};
typedef unused o0, o1, o2, o3, i1, i2, i3;
constexpr bool reverse_order = false;
constexpr bool input_evict[4] = {false, false, false, false};
__device__ void elementwise_op(size_t element_idx, int sideband, o0 &out0, o1 &out1, o2 &out2, o3 &out3,
                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {}
#define CUSTOM_VECTOR_OP
__device__ __forceinline__ void vector_op(size_type vec_idx, int vec_size, o0 *out0, o1 *out1, o2 *out2, o3 *out3,
                                          const i0 *in0, const i1 *in1, const i2 *in2, const i3 *in3,
                                          int* sideband_memory, int sideband_value) {
    // the loads must not be dead code: a value that never occurs would be reported
    if ((in0[0] ^ in0[1] ^ in0[2] ^ in0[3]) == sideband_value) sideband_memory[0] = 1;
}
"""


def cache_probe():
    """What do the caches keep of data that was only read?  A read-only op over the same buffer
    again and again, against the same op cycling through 2 GiB, for plain and nontemporal loads."""
    import torch
    from l2_torch_alloc_amd import wrapper
    lib, stream = _abi()
    big = torch.randint(0, 255, (2 * GiB,), dtype=torch.uint8, device="cuda")
    flag = torch.zeros(4, dtype=torch.int32, device="cuda")
    out = {}
    for streaming in (0, 1):
        kid = wrapper.sideaware_create_kernel((READ_ONLY_HEADER % ("nt" if streaming else "plain", streaming)).encode())
        for mib in (32, 64, 128, 256, 512):
            n = mib * MiB
            base = big.data_ptr()

            def same():
                lib.sideaware_elementwise(kid, n, 0, 0, 0, 0, base, 0, 0, 0, flag.data_ptr(), -1, 0, 0, 0, stream)

            def cycle():
                for c in range(2 * GiB // n):
                    lib.sideaware_elementwise(kid, n, 0, 0, 0, 0, base + c * n, 0, 0, 0, flag.data_ptr(), -1, 0, 0, 0,
                                              stream)

            t_same = time_region(same, 30, 3)
            t_cycle = time_region(cycle, 3, 1) / (2 * GiB // n)
            out["read_%dMiB_%s" % (mib, "nt" if streaming else "plain")] = {
                "same_buffer_GBps": gbps(n, t_same), "cycling_GBps": gbps(n, t_cycle)}
    assert int(flag[0]) == 0          # bytes are 0..254, so four equal all-ones words cannot occur
    return out


def inflight_ab(steps):
    """A/B for the question "would more loads in flight help?", meant to be run under
    `rocprofv3 --pmc TCC_EA0_RDREQ_sum TCC_EA0_RDREQ_LEVEL_sum TCC_CYCLE_sum`: the 1 GiB copy (both
    sides streaming) with 1, 2, 4 and 8 sixteen-byte loads in flight per lane.  The kernel names
    carry UNROLLED; RDREQ_LEVEL / RDREQ is the average latency of a read request at the L2's
    memory-side port."""
    import torch
    from l2_torch_alloc_amd import headers, wrapper
    lib, stream = _abi()
    n = GiB
    pairs = [(torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda"), torch.empty(n, dtype=torch.uint8, device="cuda"))
             for _ in range(2)]
    base = headers.memcpy_header().decode()
    out = {}
    for unrolled in (1, 2, 4, 8):
        text = "#define UNROLLED %d\n" % unrolled + base.replace("#define KERNEL_NAME ", "#define KERNEL_NAME unrolled%d_" % unrolled)
        kid = wrapper.sideaware_create_kernel(text.encode())

        def cycle():
            for src, dst in pairs:
                lib.sideaware_elementwise(kid, n, dst.data_ptr(), 0, 0, 0, src.data_ptr(), 0, 0, 0, 0, 0, 0, 0, 0, stream)

        sec = time_region(cycle, steps, 2) / len(pairs)
        out["unrolled_%d" % unrolled] = {"us": sec * 1e6, "GBps": gbps(2 * n, sec)}
    return out


# ------------------------------------------------------------------------------------- ceilings

NT_LOADS, NT_STORES, LANE_CONTIGUOUS, WAIT_STORES, PREFETCH, SPLIT_ROLES = 1, 2, 4, 8, 16, 32


CEILING_SOURCE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "bench_ceiling_kernels.hip")
CEILING_LIBRARY = os.path.join(os.path.dirname(os.path.abspath(__file__)), "bench_ceiling_kernels.so")


def build_ceiling_library(force=False):
    """Compiles the framework-free streaming kernels (bench_ceiling_kernels.hip) for gfx950 with
    hipcc, in-tree, when the built file is missing or older than its source."""
    import shutil
    import subprocess
    if not force and os.path.exists(CEILING_LIBRARY) and os.path.getmtime(CEILING_LIBRARY) >= os.path.getmtime(CEILING_SOURCE):
        return CEILING_LIBRARY
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    cmd = [hipcc, "--offload-arch=gfx950", "-std=c++17", "-O3", "-fPIC", "-shared",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-fvisibility=hidden",
           CEILING_SOURCE, "-o", CEILING_LIBRARY + ".tmp"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + proc.stderr)
    os.replace(CEILING_LIBRARY + ".tmp", CEILING_LIBRARY)
    return CEILING_LIBRARY


def ceiling_library():
    """The framework-free streaming kernels (bench_ceiling_kernels.hip), built on demand and bound
    with ctypes: measurement support for `bench.py --ceiling`, no part of the library."""
    path = build_ceiling_library()
    lib = ctypes.CDLL(path)
    vp, sz, ci = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
    lib.hbm_ceiling_tile.argtypes = [vp, vp, sz, ci, ci, ci, ci, vp, vp, vp]
    lib.hbm_ceiling_tile.restype = ci
    lib.hbm_ceiling_policy.argtypes = [vp, vp, sz, ci, ctypes.c_char_p, ctypes.c_char_p, ci, vp, vp]
    lib.hbm_ceiling_policy.restype = ci
    lib.hbm_ceiling_balanced_copy.argtypes = [vp, vp, sz, ci, ctypes.POINTER(ci), ctypes.POINTER(ci), vp, vp]
    lib.hbm_ceiling_balanced_copy.restype = ci
    lib.hbm_ceiling_persistent.argtypes = [vp, vp, sz, ci, ci, ci, ci, ctypes.c_uint, vp, vp]
    lib.hbm_ceiling_persistent.restype = ci
    lib.hbm_ceiling_last_error.restype = ctypes.c_char_p
    return lib


def ceiling(steps, nbytes=GiB, pairs=2, only=None):
    """What the memory system gives the simplest possible loops, none of whose operands can be
    cache-resident (launches cycle over `pairs` distinct source and destination buffers of `nbytes`
    each): read-only, write-only, independent read and write streams side by side, copies in every
    launch shape, copies in place, and copies whose read and write bursts are lined up across the
    whole chip by the device clock.  The library's own copy runs over the same buffers for
    comparison.  GB/s counts bytes read plus bytes written."""
    import torch
    lib, stream = _abi()
    ceil = ceiling_library()
    srcs = [torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device="cuda") for _ in range(pairs)]
    dsts = [torch.empty(nbytes, dtype=torch.uint8, device="cuda") for _ in range(pairs)]
    sink = torch.zeros(4, dtype=torch.int32, device="cuda")
    out = {}

    def run(name, moved, launch):
        if only and not any(o in name for o in only):
            return

        def cycle():
            for i in range(pairs):
                rc = launch(dsts[i].data_ptr(), srcs[i].data_ptr())
                assert rc in (0, None), ceil.hbm_ceiling_last_error()

        sec = time_region(cycle, steps, 2) / pairs
        out[name] = {"us": round(sec * 1e6, 2), "GBps": round(gbps(moved, sec), 1),
                     "frac_of_peak": round(gbps(moved, sec) / HBM_PEAK_GBPS, 4)}
        log("%-58s %9.1f us %8.1f GB/s" % (name, sec * 1e6, gbps(moved, sec)))

    def tile(k, block, r, flags, read=True, write=True, in_place=False):
        def launch(d, s):
            return ceil.hbm_ceiling_tile(s if in_place else (d if write else None), s if read else None,
                                         nbytes, k, block, r, flags, sink.data_ptr(), None, stream)
        return launch

    def persistent(k, block, grid, flags, period, read=True, write=True):
        def launch(d, s):
            return ceil.hbm_ceiling_persistent(d if write else None, s if read else None, nbytes, k, block, grid,
                                               flags, period, sink.data_ptr(), stream)
        return launch

    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipMemsetAsync.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_void_p]
    hip.hipMemsetAsync.restype = ctypes.c_int
    hip.hipMemcpyAsync.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p]
    hip.hipMemcpyAsync.restype = ctypes.c_int
    by_ptr = {t.data_ptr(): t for t in srcs + dsts}

    hints = {"plain": 0, "nt": NT_LOADS | NT_STORES}
    run("library sideaware_memcpy", 2 * nbytes, lambda d, s: lib.sideaware_memcpy(d, s, nbytes, 0, stream))
    run("vendor copy: hipMemcpyAsync device to device", 2 * nbytes, lambda d, s: hip.hipMemcpyAsync(d, s, nbytes, 3, stream))
    run("vendor copy: torch copy_", 2 * nbytes, lambda d, s: (by_ptr[d].copy_(by_ptr[s]), None)[1])
    run("vendor write-only: hipMemsetAsync", nbytes, lambda d, s: hip.hipMemsetAsync(d, 1, nbytes, stream))
    run("vendor write-only: torch fill_", nbytes, lambda d, s: (by_ptr[d].fill_(3), None)[1])
    for hint, f in hints.items():
        for k in (1, 4):
            run("read-only tile k=%d block=256 %s" % (k, hint), nbytes, tile(k, 256, 2, f, write=False))
            run("write-only tile k=%d block=256 %s" % (k, hint), nbytes, tile(k, 256, 2, f, read=False))
        run("read-only persistent k=8 block=1024 grid=512 %s" % hint, nbytes,
            persistent(8, 1024, 512, f, 0, write=False))
        for k, block, grid in ((8, 1024, 512), (4, 256, 2048), (1, 256, 2048), (1, 256, 8192), (1, 64, 8192)):
            run("write-only persistent k=%d block=%d grid=%d %s" % (k, block, grid, hint), nbytes,
                persistent(k, block, grid, f, 0, read=False))
        for k, block, r in ((1, 64, 0), (1, 128, 0), (1, 512, 0), (1, 1024, 0), (2, 256, 0), (1, 256, 0), (1, 256, 4),
                            (1, 256, 7)):
            run("write-only tile k=%d block=%d stripe=%dKiB %s" % (k, block, (k * block * 16 << r) >> 10, hint), nbytes,
                tile(k, block, r, f, read=False))
        run("independent read and write streams, tile k=1 block=256 %s" % hint, nbytes,
            tile(1, 256, 2, f | SPLIT_ROLES))
    for k, block, r in ((1, 256, 0), (1, 256, 2), (2, 256, 1), (4, 256, 0), (8, 256, 0), (1, 1024, 0), (4, 1024, 0),
                        (8, 1024, 0), (16, 1024, 0)):
        run("copy tile k=%d block=%d stripe=%dKiB nt" % (k, block, (k * block * 16 << r) >> 10), 2 * nbytes,
            tile(k, block, r, hints["nt"]))
    for k in (2, 4):
        run("copy tile k=%d block=256 lane-contiguous nt" % k, 2 * nbytes,
            tile(k, 256, 0, hints["nt"] | LANE_CONTIGUOUS))
    run("copy tile k=1 block=256 loads nt, stores plain", 2 * nbytes, tile(1, 256, 2, NT_LOADS))
    run("copy tile k=1 block=256 loads plain, stores nt", 2 * nbytes, tile(1, 256, 2, NT_STORES))
    for k in (1, 2):
        run("copy in place tile k=%d block=256 nt" % k, 2 * nbytes, tile(k, 256, 2, hints["nt"], in_place=True))
    for k, block, grid in ((8, 1024, 256), (8, 1024, 512), (16, 1024, 256), (8, 256, 2048), (16, 256, 1024),
                           (2, 256, 4096), (1, 256, 8192)):
        for wait in (0, WAIT_STORES):
            run("copy persistent bursts k=%d block=%d grid=%d%s nt" % (k, block, grid, " wait-stores" if wait else ""),
                2 * nbytes, persistent(k, block, grid, hints["nt"] | wait, 0))
    # persistent grids again, software-pipelined: the next chunk's loads are issued before the
    # current chunk's stores (flag 16), beside the same grid without
    for k, block, grid in ((1, 256, 1024), (1, 256, 2048), (2, 256, 1024), (2, 256, 2048), (4, 256, 1024),
                           (1, 256, 4096), (2, 256, 4096), (1, 1024, 512), (2, 1024, 256)):
        for prefetch in (0, 16):
            run("copy persistent%s k=%d block=%d grid=%d nt" % (" prefetch" if prefetch else " no-prefetch", k, block, grid),
                2 * nbytes, persistent(k, block, grid, hints["nt"] | prefetch, 0))
    # the workgroup -> address map: stripes of 2^r tiles per XCD, from tile-by-tile round robin (r = 0:
    # consecutive workgroups take consecutive 4 KiB chunks) to 2 MiB runs per XCD
    for r in range(0, 10):
        kib = 4 << r
        run("stripe sweep: read-only k=1 block=256 stripe=%dKiB nt" % kib, nbytes, tile(1, 256, r, hints["nt"], write=False))
        run("stripe sweep: write-only k=1 block=256 stripe=%dKiB nt" % kib, nbytes, tile(1, 256, r, hints["nt"], read=False))
        run("stripe sweep: write-only k=1 block=256 stripe=%dKiB plain" % kib, nbytes, tile(1, 256, r, 0, read=False))
        run("stripe sweep: independent streams k=1 block=256 stripe=%dKiB nt" % kib, nbytes,
            tile(1, 256, r, hints["nt"] | SPLIT_ROLES))
        run("stripe sweep: copy k=1 block=256 stripe=%dKiB nt" % kib, 2 * nbytes, tile(1, 256, r, hints["nt"]))
        run("stripe sweep: copy in place k=1 block=256 stripe=%dKiB nt" % kib, 2 * nbytes,
            tile(1, 256, r, hints["nt"], in_place=True))
    for stripe in (4096, 8192, 16384, 32768, 65536, 262144, 524288, 2097152):
        assert lib.sideaware_tune(b"stripe_bytes", stripe) == 0
        run("stripe sweep: library sideaware_memcpy stripe_bytes=%d" % stripe, 2 * nbytes,
            lambda d, s: lib.sideaware_memcpy(d, s, nbytes, 0, stream))
    assert lib.sideaware_tune(b"stripe_bytes", 0) == 0
    # time against size, per stripe: a straight-line fit separates the steady rate from the cost of
    # starting and draining a launch
    if only and any("size fit" in o for o in only):
        big_src = torch.empty(4 * GiB, dtype=torch.uint8, device="cuda")
        big_src.view(torch.int64).random_()
        big_dst = torch.empty(4 * GiB, dtype=torch.uint8, device="cuda")
        for r in (0, 2, 5, 6, 7, 8, 9):
            for mib in (64, 128, 256, 512, 1024, 2048):
                size, slots = mib * MiB, (4 * GiB) // (mib * MiB)

                def cycle():
                    for j in range(slots):
                        rc = ceil.hbm_ceiling_tile(big_dst.data_ptr() + j * size, big_src.data_ptr() + j * size, size,
                                                   1, 256, r, hints["nt"], sink.data_ptr(), None, stream)
                        assert rc == 0

                sec = time_region(cycle, max(2, steps // 2), 1) / slots
                name = "size fit: copy k=1 block=256 stripe=%dKiB nt size=%dMiB" % (4 << r, mib)
                out[name] = {"us": round(sec * 1e6, 2), "GBps": round(gbps(2 * size, sec), 1)}
                log("%-58s %9.1f us %8.1f GB/s" % (name, sec * 1e6, gbps(2 * size, sec)))
        del big_src, big_dst
    # the cache-policy bits of loads and stores, spelled out in the instructions
    if only and any("policy bits" in o for o in only):
        bits = ("", "nt", "sc1", "sc0 sc1", "sc1 nt", "sc0 sc1 nt", "sc0")
        r = 8 if nbytes >= 512 * MiB else 5

        def policy(loads, stores, mode):
            def launch(d, s_):
                return ceil.hbm_ceiling_policy(d, s_, nbytes, r, loads.encode(), stores.encode(), mode, sink.data_ptr(), stream)
            return launch

        for rnd in range(2):
            for lb in bits:
                run("policy bits: read-only, loads '%s' (round %d)" % (lb, rnd), nbytes, policy(lb, "", 1))
            for sb in bits:
                run("policy bits: write-only, stores '%s' (round %d)" % (sb, rnd), nbytes, policy("", sb, 2))
            for lb in bits:
                for sb in bits:
                    run("policy bits: copy, loads '%s', stores '%s' (round %d)" % (lb, sb, rnd), 2 * nbytes, policy(lb, sb, 0))
    # unequal shares per XCD: measure how far ahead of the last XCD each one finishes, give the slow
    # ones fewer tiles and the fast ones more, and time the copy again
    if only and any("xcd shares" in o for o in only):
        import numpy as np
        for size_mib, r in ((256, 5), (1024, 8)):
            size = size_mib * MiB
            own = size // 4096 // 8
            ci8 = ctypes.c_int * 8
            equal_cut, zero = ci8(*([own] * 8)), ci8(*([0] * 8))

            def measure_leads(cut, extra, reps=10):
                slots = own + max(extra)
                stamps = torch.zeros(2 * 8 * slots, dtype=torch.int64, device="cuda")
                leads, spans = [], []
                for rep in range(reps):
                    i = rep % pairs
                    stamps.zero_()
                    torch.cuda.synchronize()
                    rc = ceil.hbm_ceiling_balanced_copy(dsts[i].data_ptr(), srcs[i].data_ptr(), size, r, cut, extra,
                                                        stamps.data_ptr(), stream)
                    assert rc == 0, ceil.hbm_ceiling_last_error()
                    torch.cuda.synchronize()
                    assert bool(torch.equal(dsts[i][:size], srcs[i][:size]))
                    t = stamps.view(8 * slots, 2)
                    ran = t[:, 1] != 0
                    ends = np.array([int(t[x::8, 1].max()) for x in range(8)], dtype=np.int64)
                    start = int(t[:, 0][ran].min())
                    if rep >= 2:
                        leads.append((ends.max() - ends) / 100.0)
                        spans.append((ends.max() - start) / 100.0)
                return np.mean(leads, axis=0), float(np.mean(spans))

            def timed(cut, extra):
                def cycle():
                    for i in range(pairs):
                        rc = ceil.hbm_ceiling_balanced_copy(dsts[i].data_ptr(), srcs[i].data_ptr(), size, r, cut, extra,
                                                            None, stream)
                        assert rc == 0
                return time_region(cycle, max(steps, 6), 2) / pairs

            leads, span = measure_leads(equal_cut, zero)
            speed = own / (span - leads)                     # tiles per us of each XCD
            want = np.floor(speed / speed.sum() * own * 8 + 0.5).astype(int)
            want[int(np.argmax(want))] += own * 8 - int(want.sum())
            cut = ci8(*[int(min(own, w)) for w in want])
            extra = ci8(*[int(max(0, w - own)) for w in want])
            leads2, span2 = measure_leads(cut, extra)
            t_equal = [timed(equal_cut, zero), None, None]
            t_shares = [timed(cut, extra), None, None]
            for j in (1, 2):
                t_equal[j] = timed(equal_cut, zero)
                t_shares[j] = timed(cut, extra)
            name = "xcd shares: copy %dMiB stripe=%dKiB nt" % (size_mib, 4 << r)
            out[name] = {"equal_shares_us": [round(x * 1e6, 2) for x in t_equal],
                         "measured_shares_us": [round(x * 1e6, 2) for x in t_shares],
                         "equal_GBps": round(gbps(2 * size, min(t_equal)), 1),
                         "measured_shares_GBps": round(gbps(2 * size, min(t_shares)), 1),
                         "tiles_per_xcd": [int(w) for w in want], "own": own,
                         "leads_us_equal": [round(float(x), 2) for x in leads], "span_us_equal": round(span, 2),
                         "leads_us_shares": [round(float(x), 2) for x in leads2], "span_us_shares": round(span2, 2)}
            log(name, out[name])
    # the same launches spread over two streams: a launch may start while the one before it drains
    if only and any("two streams" in o for o in only):
        n = 256 * MiB
        k_pairs = 8
        s_srcs = [torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda") for _ in range(k_pairs)]
        s_dsts = [torch.empty(n, dtype=torch.uint8, device="cuda") for _ in range(k_pairs)]
        side = [torch.cuda.Stream(), torch.cuda.Stream()]
        for st in side:                               # streams are made on first use: not inside a timed region
            st.wait_stream(torch.cuda.current_stream())
            torch.cuda.current_stream().wait_stream(st)
        torch.cuda.synchronize()
        for label, streams in (("one stream", [torch.cuda.current_stream()]), ("two streams", side)):
            for i in range(k_pairs):                  # untimed: every stream and buffer has been used once
                lib.sideaware_memcpy(s_dsts[i].data_ptr(), s_srcs[i].data_ptr(), n, 0, streams[i % len(streams)].cuda_stream)
            torch.cuda.synchronize()
            ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            reps = 6
            ev0.record()
            for st in side:
                st.wait_event(ev0)
            for rep in range(reps):
                for i in range(k_pairs):
                    st = streams[i % len(streams)]
                    lib.sideaware_memcpy(s_dsts[i].data_ptr(), s_srcs[i].data_ptr(), n, 0, st.cuda_stream)
            for st in side:
                torch.cuda.current_stream().wait_stream(st)
            ev1.record()
            torch.cuda.synchronize()
            sec = ev0.elapsed_time(ev1) * 1e-3 / (reps * k_pairs)
            name = "two streams: library copy 256MiB x 8 pairs, launches on %s" % label
            out[name] = {"us": round(sec * 1e6, 2), "GBps": round(gbps(2 * n, sec), 1)}
            log("%-58s %9.1f us %8.1f GB/s" % (name, sec * 1e6, gbps(2 * n, sec)))
        assert all(bool(torch.equal(d, t)) for d, t in zip(s_dsts, s_srcs))
        del s_srcs, s_dsts
    # when does each XCD start and finish its share of a launch?  (device clock, 10 ns ticks; every
    # workgroup writes its own start and end time, the host reduces them per XCD: workgroup i runs on XCD i % 8)
    if only and any("xcd spread" in o for o in only):
        for size_mib, r in ((256, 5), (256, 8), (1024, 8), (64, 5)):
            size = size_mib * MiB
            tiles = size // 4096
            stamps = torch.zeros(2 * tiles, dtype=torch.int64, device="cuda")
            finish, start, durs, ramp = [], [], [], []
            for rep in range(10):
                i = rep % pairs
                torch.cuda.synchronize()
                rc = ceil.hbm_ceiling_tile(dsts[i].data_ptr(), srcs[i].data_ptr(), size, 1, 256, r, hints["nt"],
                                           sink.data_ptr(), stamps.data_ptr(), stream)
                assert rc == 0
                torch.cuda.synchronize()
                t = stamps.view(tiles, 2)
                t0 = torch.stack([t[x::8, 0].min() for x in range(8)]).cpu().numpy()
                t1 = torch.stack([t[x::8, 1].max() for x in range(8)]).cpu().numpy()
                first_done = int(t[:, 1].min())
                if rep >= 2:
                    log("   rep %d pair %d: per-XCD finish, us before the last one: %s" % (
                        rep, i, " ".join("%5.2f" % ((int(t1.max()) - int(v)) / 100.0) for v in t1)))
                    finish.append((int(t1.max()) - int(t1.min())) / 100.0)
                    start.append((int(t0.max()) - int(t0.min())) / 100.0)
                    durs.append((int(t1.max()) - int(t0.min())) / 100.0)
                    ramp.append((first_done - int(t0.min())) / 100.0)
            name = "xcd spread: copy %dMiB stripe=%dKiB nt" % (size_mib, 4 << r)
            out[name] = {"first_start_to_last_end_us": round(sum(durs) / len(durs), 2),
                         "last_minus_first_xcd_to_finish_us": round(sum(finish) / len(finish), 2),
                         "worst_us": round(max(finish), 2),
                         "last_minus_first_xcd_to_start_us": round(sum(start) / len(start), 2),
                         "first_workgroup_done_after_us": round(sum(ramp) / len(ramp), 2)}
            log(name, out[name])
            del stamps
    # chip-wide phases: one iteration of the whole grid moves grid*block*k*16 bytes each way; the
    # period is swept around the time that takes at 6.2-7.2 TB/s
    for k, block, grid in ((16, 1024, 256), (8, 1024, 512), (8, 1024, 256)):
        per_iter = 2 * grid * block * k * 16
        for tbps in (6.0, 6.4, 6.8, 7.2):
            ticks = int(round(per_iter / (tbps * 1e12) * 1e8))          # 100 MHz clock
            for wait in (0, WAIT_STORES):
                run("copy clock-phased k=%d block=%d grid=%d period=%.2fus%s nt" % (
                    k, block, grid, ticks / 100.0, " wait-stores" if wait else ""),
                    2 * nbytes, persistent(k, block, grid, hints["nt"] | wait, ticks))
    torch.cuda.synchronize()
    assert int(sink[0]) == 0
    return out


# ------------------------------------------------------------------------------------- launch shapes

def launch_shapes(steps, only=None):
    """The library's own kernels under the never-cached protocol (launches cycle over distinct
    buffer sets), for every ownership stripe from 4 KiB to 2 MiB: the copy at 64 MiB, 256 MiB and
    1 GiB, and the in-place bf16 RoPE of the Llama-3-8B step (q, then k) with 4 KiB and 8 KiB tiles."""
    import torch
    from l2_torch_alloc_amd import headers, ops, wrapper
    lib, stream = _abi()
    out = {}
    stripes = (4096, 16384, 65536, 131072, 262144, 524288, 1048576, 2097152)
    # let the stripe be what the sweep says even for the smaller arrays (the library otherwise
    # shrinks it until every XCD owns at least 32 stripes)
    assert lib.sideaware_tune(b"stripes_per_xcd", 2) == 0

    def want(name):
        return not only or any(o in name for o in only)

    for nbytes, pairs in ((16 * MiB, 64), (64 * MiB, 16), (256 * MiB, 8), (GiB, 2), (4 * GiB, 1)):
        if not want("copy %dMiB" % (nbytes // MiB)):
            continue
        srcs = [torch.empty(nbytes, dtype=torch.uint8, device="cuda") for _ in range(pairs)]
        for t in srcs:
            t.view(torch.int64).random_()
        dsts = [torch.empty(nbytes, dtype=torch.uint8, device="cuda") for _ in range(pairs)]
        ptrs = [(d.data_ptr(), s.data_ptr()) for d, s in zip(dsts, srcs)]

        def cycle():
            for d, s in ptrs:
                lib.sideaware_memcpy(d, s, nbytes, 0, stream)

        for stripe in stripes:
            assert lib.sideaware_tune(b"stripe_bytes", stripe) == 0
            sec = time_region(cycle, steps, 2) / pairs
            name = "copy %dMiB x %d pairs stripe_bytes=%d" % (nbytes // MiB, pairs, stripe)
            out[name] = {"us": round(sec * 1e6, 2), "GBps": round(gbps(2 * nbytes, sec), 1)}
            log("%-60s %9.2f us %8.1f GB/s" % (name, sec * 1e6, gbps(2 * nbytes, sec)))
        assert all(bool(torch.equal(d, s)) for d, s in zip(dsts, srcs))
        del srcs, dsts

    if want("rope"):
        B, T, HS, sets = 8, 4096, 128, 5
        freqs = ops.freqs_cis_table(HS, T, 500000.0).cuda()
        qs = [torch.randn(B, T, 32, HS, device="cuda").to(torch.bfloat16) for _ in range(sets)]
        ks = [torch.randn(B, T, 8, HS, device="cuda").to(torch.bfloat16) for _ in range(sets)]
        q_bytes, k_bytes, fp = qs[0].numel() * 2, ks[0].numel() * 2, freqs.data_ptr()
        total = 2 * (q_bytes + k_bytes) + freqs.numel() * 4
        for unrolled in (1, 2, 4):
            kid_q = wrapper.sideaware_create_kernel(headers.rope_header(T, 32, 0, HS, "bf16", "heads", unrolled=unrolled))
            kid_k = wrapper.sideaware_create_kernel(headers.rope_header(T, 8, 0, HS, "bf16", "heads", unrolled=unrolled))

            def cycle():
                for q, k in zip(qs, ks):
                    lib.sideaware_elementwise(kid_q, q_bytes, q.data_ptr(), 0, 0, 0, q.data_ptr(), fp, 0, 0, 0, 0, 0, 0, 0, stream)
                    lib.sideaware_elementwise(kid_k, k_bytes, k.data_ptr(), 0, 0, 0, k.data_ptr(), fp, 0, 0, 0, 0, 0, 0, 0, stream)

            for stripe in stripes:
                assert lib.sideaware_tune(b"stripe_bytes", stripe) == 0
                sec = time_region(cycle, steps, 2) / sets
                name = "rope bf16 q+k x %d sets tile=%dKiB stripe_bytes=%d" % (sets, 4 * unrolled, stripe)
                out[name] = {"us": round(sec * 1e6, 2), "GBps": round(gbps(total, sec), 1)}
                log("%-60s %9.2f us %8.1f GB/s" % (name, sec * 1e6, gbps(total, sec)))
        # larger workgroups (a compiled-in knob: every kernel is built afresh for it), 4 KiB per workgroup instruction
        # becomes 8 or 16 KiB
        for wg in (512, 1024):
            assert lib.sideaware_tune(b"wg_threads", wg) == 0 and lib.sideaware_tune(b"stripe_bytes", 0) == 0
            for unrolled in (1, 2):
                if wg * unrolled * 16 > 16384:
                    continue
                kid_q = wrapper.sideaware_create_kernel(headers.rope_header(T, 32, 0, HS, "bf16", "heads", unrolled=unrolled))
                kid_k = wrapper.sideaware_create_kernel(headers.rope_header(T, 8, 0, HS, "bf16", "heads", unrolled=unrolled))

                def cycle_wg():
                    for q, k in zip(qs, ks):
                        lib.sideaware_elementwise(kid_q, q_bytes, q.data_ptr(), 0, 0, 0, q.data_ptr(), fp, 0, 0, 0, 0, 0, 0, 0, stream)
                        lib.sideaware_elementwise(kid_k, k_bytes, k.data_ptr(), 0, 0, 0, k.data_ptr(), fp, 0, 0, 0, 0, 0, 0, 0, stream)

                sec = time_region(cycle_wg, steps, 2) / sets
                name = "rope bf16 q+k x %d sets workgroup=%d threads tile=%dKiB stripe by size" % (sets, wg, wg * unrolled * 16 // 1024)
                out[name] = {"us": round(sec * 1e6, 2), "GBps": round(gbps(total, sec), 1)}
                log("%-60s %9.2f us %8.1f GB/s" % (name, sec * 1e6, gbps(total, sec)))
        assert lib.sideaware_tune(b"wg_threads", 256) == 0
        # q and k in one launch (one kernel, the head count travels in the sideband value)
        for unrolled in (1, 2):
            kid = wrapper.sideaware_create_kernel(headers.rope_header(T, 0, 0, HS, "bf16", "heads", unrolled=unrolled,
                                                                      heads_at_launch=True))
            batches = []
            for q, k in zip(qs, ks):
                arr = (ops._Segment * 2)()
                for seg, t in zip(arr, (q, k)):
                    seg.num_bytes = t.numel() * 2
                    seg.out[0] = t.data_ptr()
                    seg.inp[0] = t.data_ptr()
                    seg.inp[1] = fp
                    seg.sideband_value = t.shape[2]
                batches.append(arr)

            def cycle_batched():
                for arr in batches:
                    lib.sideaware_elementwise_batch(kid, 2, arr, 0, stream)

            for stripe in (0,) + stripes:
                assert lib.sideaware_tune(b"stripe_bytes", stripe) == 0
                sec = time_region(cycle_batched, steps, 2) / sets
                name = "rope bf16 q+k in one launch x %d sets tile=%dKiB stripe_bytes=%d" % (sets, 4 * unrolled, stripe)
                out[name] = {"us": round(sec * 1e6, 2), "GBps": round(gbps(total, sec), 1)}
                log("%-60s %9.2f us %8.1f GB/s" % (name, sec * 1e6, gbps(total, sec)))
    assert lib.sideaware_tune(b"stripe_bytes", 0) == 0 and lib.sideaware_tune(b"stripes_per_xcd", 8) == 0
    return out


# ------------------------------------------------------------------------------------- producer -> consumer, per XCD

def chain_xcd(reps=4, only=None):
    """Producer -> consumer on the same buffer, meant to be run under `rocprofv3 --pmc` with the per-XCD
    TCC_HIT / TCC_MISS counters of profiles/xcd_counters.yaml: a copy writes `mid`, and at once a
    second copy reads `mid`, walking each XCD's tiles in the same order or in reverse
    (`reverse_order`, the reference's knob for exactly this: sideaware.cu:40), so that it starts with
    what the producer wrote last.  The producer's stores are the library's two policies, `sc1`
    (written through the private L2, left cacheable) and `sc1nt` (the same, streaming), or, for
    comparison, the same stores without the scope bit (`plain`, `nt`).  Buffer sets cycle, so nothing
    but the producer's result can be cache-resident.  Kernel names carry size, store policy and
    order; per-launch times come from HIP events."""
    import torch
    from l2_torch_alloc_amd import headers, wrapper
    lib, stream = _abi()
    base = headers.memcpy_header().decode()
    out = {}

    store_defines = {"sc1": "#define OUTPUT_STREAMING 0\n", "sc1nt": "#define OUTPUT_STREAMING 1\n",
                     "plain": '#define SA_STORE_POLICY ""\n', "nt": '#define SA_STORE_POLICY "nt"\n'}

    def kernel(tag, stores, reverse, stream_in=1):
        text = "#define INPUT0_STREAMING %d\n" % stream_in + store_defines[stores] + base
        text = text.replace("#define KERNEL_NAME ", "#define KERNEL_NAME " + tag)
        text = text.replace("constexpr bool reverse_order = false;", "constexpr bool reverse_order = %s;" % ("true" if reverse else "false"))
        return wrapper.sideaware_create_kernel(text.encode())

    for mib in (8, 32, 64, 128, 256, 512):
        nbytes = mib * MiB
        sets = min(24, max(3, (1536 * MiB) // (3 * nbytes)))
        srcs = [torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device="cuda") for _ in range(sets)]
        mids = [torch.empty_like(t) for t in srcs]
        outs = [torch.empty_like(t) for t in srcs]
        # the consumer's loads carry the streaming hint, except in the "plainloads" cases
        cases = [(policy, order, 1) for policy in ("sc1", "sc1nt") for order in ("same", "reversed")]
        cases += [("plain", "same", 1), ("nt", "same", 1), ("sc1", "same", 0), ("sc1", "reversed", 0)]
        for policy, order, consumer_stream_in in cases:
                reverse = order == "reversed"
                name = "%dMiB_%s_%s%s" % (mib, policy, order, "" if consumer_stream_in else "_plainloads")
                if only and not any(o in name for o in only):
                    continue
                producer = kernel("chainP_%s_" % name, policy, False)
                consumer = kernel("chainC_%s_" % name, "sc1nt", reverse, consumer_stream_in)
                evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(sets)]
                tp = tc = 0.0
                for rep in range(reps + 1):
                    for i in range(sets):
                        e = evs[i]
                        e[0].record()
                        lib.sideaware_one_to_one(producer, nbytes, mids[i].data_ptr(), srcs[i].data_ptr(), 0, stream)
                        e[1].record()
                        lib.sideaware_one_to_one(consumer, nbytes, outs[i].data_ptr(), mids[i].data_ptr(), 0, stream)
                        e[2].record()
                    torch.cuda.synchronize()
                    if rep:
                        tp += sum(e[0].elapsed_time(e[1]) for e in evs)
                        tc += sum(e[1].elapsed_time(e[2]) for e in evs)
                n = reps * sets
                ok = all(bool(torch.equal(o, s)) for o, s in zip(outs, srcs))
                out[name] = {"producer_us": round(tp / n * 1e3, 2), "consumer_us": round(tc / n * 1e3, 2),
                             "consumer_GBps": round(gbps(2 * nbytes, tc / n * 1e-3), 1), "sets": sets, "bit_exact": ok}
                log("%-28s producer %8.2f us  consumer %8.2f us (%7.1f GB/s)  %s" % (
                    name, tp / n * 1e3, tc / n * 1e3, gbps(2 * nbytes, tc / n * 1e-3), "ok" if ok else "WRONG"))
        del srcs, mids, outs
    return out
