"""The allocator on a real device, through PyTorch's pluggable-allocator hooks and through the
direct C entry points (sideaware.cu:1280-1352 are the reference's versions)."""
import ctypes
import random

import pytest
import torch

pytestmark = pytest.mark.gpu

MiB = 1 << 20


def test_torch_tensors_come_from_the_pool(sa):
    before = sa.sideaware_alloc_stats()
    big = torch.empty(24 * MiB, dtype=torch.uint8, device="cuda")
    small = torch.empty(1000, dtype=torch.uint8, device="cuda")
    after = sa.sideaware_alloc_stats()
    assert big.data_ptr() % (2 * MiB) == 0
    assert small.data_ptr() % 512 == 0
    large = lambda st: st["large_hits"] + st["large_misses"] + st["large_carves"]
    assert large(after) == large(before) + 1
    assert after["small_hits"] + after["small_carves"] == before["small_hits"] + before["small_carves"] + 1
    assert after["bytes_live"] >= before["bytes_live"] + 24 * MiB + 1024


def test_same_size_blocks_share_the_stripe_phase_and_are_reused(sa):
    a = torch.empty(40 * MiB, dtype=torch.uint8, device="cuda")
    b = torch.empty(40 * MiB, dtype=torch.uint8, device="cuda")
    assert a.data_ptr() % (2 * MiB) == 0 and b.data_ptr() % (2 * MiB) == 0
    pa = a.data_ptr()
    del a
    c = torch.empty(40 * MiB - 100, dtype=torch.uint8, device="cuda")   # rounds to the same 40 MiB
    assert c.data_ptr() == pa                                             # newest freed block first


def test_direct_malloc_free(sa):
    lib = sa.library()
    p = ctypes.c_void_p()
    assert lib.sideaware_malloc(ctypes.byref(p), 3 * MiB + 5) == 0
    assert p.value and p.value % (2 * MiB) == 0
    first = p.value
    assert lib.sideaware_free(p) == 0
    q = ctypes.c_void_p()
    assert lib.sideaware_malloc_async(ctypes.byref(q), 4 * MiB, None) == 0
    assert q.value == first                                               # same rounded size: reused
    # the memory is real: fill and copy through the kernels
    r = ctypes.c_void_p()
    assert lib.sideaware_malloc_async(ctypes.byref(r), 4 * MiB, None) == 0
    host = torch.arange(MiB, dtype=torch.int32)
    dev = host.cuda()
    lib.sideaware_memcpy(q, dev.data_ptr(), 4 * MiB, 0, None)
    lib.sideaware_memcpy(r, q, 4 * MiB, 0, None)
    back = torch.zeros_like(dev)
    lib.sideaware_memcpy(back.data_ptr(), r, 4 * MiB, 0, None)
    torch.cuda.synchronize()
    assert torch.equal(back.cpu(), host)
    assert lib.sideaware_free_async(q, None) == 0
    assert lib.sideaware_free_async(r, None) == 0
    assert lib.sideaware_free_async(None, None) == 0


def test_release_unused_gives_memory_back(sa):
    lib = sa.library()
    x = torch.empty(64 * MiB, dtype=torch.uint8, device="cuda")
    del x
    torch.cuda.synchronize()
    before = sa.sideaware_alloc_stats()
    assert before["bytes_cached_large"] >= 64 * MiB
    freed = lib.sideaware_release_unused()
    after = sa.sideaware_alloc_stats()
    # the cache is folded back into the arenas and every wholly free arena returns to the driver;
    # an arena that still holds a live region stays
    assert after["bytes_cached_large"] == 0
    assert after["bytes_reserved"] == before["bytes_reserved"] - freed
    assert (after["bytes_free_arena"] + after["bytes_free_slab_arena"] + after["bytes_live"]
            + after["bytes_cached_small"]) <= after["bytes_reserved"]


def test_out_of_memory_is_a_null_pointer_for_c_callers_and_an_exception_for_pytorch(sa):
    # More than the device holds: every step of the ladder fails and the entry point returns null
    # (sideaware.cu:1250-1251 ends the same way).  PyTorch's pluggable-allocator shim does not check
    # the pointer and would build a tensor with a null data pointer, so PyTorch is given another
    # entry point (sideaware_malloc_auto_raising), which raises instead: torch.empty fails loudly.
    total = torch.cuda.get_device_properties(0).total_memory
    lib = sa.library()
    before = sa.sideaware_alloc_stats()["failures"]
    p = lib.sideaware_malloc_auto(total + (8 << 30), 0, None)      # a C caller (ctypes is one) gets null
    assert p is None
    assert sa.sideaware_alloc_stats()["failures"] == before + 1
    with pytest.raises(RuntimeError, match="sideaware: out of memory"):
        torch.empty(total + (8 << 30), dtype=torch.uint8, device="cuda")
    assert "out of memory" in sa.sideaware_last_error()
    out = ctypes.c_void_p(1)
    assert lib.sideaware_malloc(ctypes.byref(out), total + (8 << 30)) == 2      # hipErrorOutOfMemory
    assert out.value is None
    lib.sideaware_clear_error()
    # and the pool still serves requests afterwards
    y = torch.ones(10 * MiB, dtype=torch.uint8, device="cuda")
    assert int(y.sum()) == 10 * MiB


def test_reserve_limit_acts_like_a_full_device(sa):
    lib = sa.library()
    lib.sideaware_release_unused()
    st = sa.sideaware_alloc_stats()
    lib.sideaware_reserve_limit(st["bytes_reserved"] + 256 * MiB)
    try:
        ok = lib.sideaware_malloc_auto(128 * MiB, 0, None)            # free arena space, or a small new arena
        assert ok and ok % (2 * MiB) == 0
        too_much = sa.sideaware_alloc_stats()["bytes_free_arena"] + (1 << 30)
        assert lib.sideaware_malloc_auto(too_much, 0, None) is None    # would need > 256 MiB more from the driver
        assert sa.sideaware_alloc_stats()["failures"] == st["failures"] + 1
        lib.sideaware_free_auto(ok, 128 * MiB, 0, None)
    finally:
        lib.sideaware_reserve_limit(0)
        lib.sideaware_clear_error()
    z = torch.empty(512 * MiB, dtype=torch.uint8, device="cuda")
    assert z.data_ptr() % (2 * MiB) == 0


def test_regions_are_carved_from_arenas(sa):
    lib = sa.library()
    lib.sideaware_release_unused()
    before = sa.sideaware_alloc_stats()
    tensors = [torch.empty((24 + 2 * i) * MiB, dtype=torch.uint8, device="cuda") for i in range(8)]
    after = sa.sideaware_alloc_stats()
    assert all(t.data_ptr() % (2 * MiB) == 0 for t in tensors)
    # eight different sizes, at most one new arena from the driver
    assert after["backing_acquires"] - before["backing_acquires"] <= 1
    assert after["large_carves"] - before["large_carves"] >= 7
    spans = sorted((t.data_ptr(), t.data_ptr() + t.numel()) for t in tensors)
    assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:]))
    for i, t in enumerate(tensors):
        t.fill_(i + 1)
    torch.cuda.synchronize()
    assert [int(t[0]) for t in tensors] == list(range(1, 9)) and [int(t[-1]) for t in tensors] == list(range(1, 9))


def test_threshold_and_trim_settings_apply(sa):
    lib = sa.library()
    lib.sideaware_free_mapped_thresholds(32 * MiB, 0)
    try:
        blocks = [torch.empty((10 + 2 * i) * MiB, dtype=torch.uint8, device="cuda") for i in range(6)]
        del blocks
        st = sa.sideaware_alloc_stats()
        assert st["bytes_cached_large"] >= 90 * MiB
        # a request no cached region and no free extent can serve: a miss with the cache over budget
        z = torch.empty(st["bytes_free_arena"] + 64 * MiB, dtype=torch.uint8, device="cuda")
        after = sa.sideaware_alloc_stats()
        assert after["trims"] == st["trims"] + 1 and after["bytes_cached_large"] == 0
        del z
    finally:
        lib.sideaware_free_mapped_thresholds(16 << 30, 2 << 30)
    lib.sideaware_alloc_threshold(1 * MiB)
    try:
        t = torch.empty(MiB, dtype=torch.uint8, device="cuda")
        assert t.data_ptr() % (2 * MiB) == 0
    finally:
        lib.sideaware_alloc_threshold(8 * MiB)


def test_churn_contents_survive(sa):
    # tensors of random sizes filled with a tag; whatever the pool recycles, live data must stay put
    rng = random.Random(7)
    live = []
    for step in range(400):
        if live and rng.random() < 0.5:
            t, tag = live.pop(rng.randrange(len(live)))
            assert int(t[0]) == tag and int(t[-1]) == tag
        else:
            n = int(4096 * 2 ** (rng.random() * 14)) // 4
            tag = step
            t = torch.full((n,), tag, dtype=torch.int32, device="cuda")
            live.append((t, tag))
    for t, tag in live:
        assert bool((t == tag).all())


def test_memcpy_under_torch_compile(sa):
    # the custom op traces with fullgraph=True (test.py:175-184)
    @torch.compile(fullgraph=True)
    def compiled_copy(dst, src):
        torch.ops.sideaware.memcpy(dst, src)
        return dst

    src = torch.ones((8, 8), dtype=torch.float32, device="cuda") * 2.0
    dst = torch.zeros((8, 8), dtype=torch.float32, device="cuda")
    out = compiled_copy(dst, src)
    torch.cuda.synchronize()
    assert torch.equal(out, src) and torch.equal(dst, src)


def test_block_handed_to_another_stream_waits_for_the_first(sa):
    # Stream order (sideaware.cu:1209-1212): a block freed on stream A while A still has work
    # queued on it, then handed to stream B, must not be touched by B before A is done with it.
    lib = sa.library()
    n = 256 * MiB
    ones = torch.full((n,), 1, dtype=torch.uint8, device="cuda")
    twos = torch.full((n,), 2, dtype=torch.uint8, device="cuda")
    result = torch.zeros(n, dtype=torch.uint8, device="cuda")
    a, b = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    before = sa.sideaware_alloc_stats()
    p = lib.sideaware_malloc_auto(n, 0, a.cuda_stream)
    assert p
    for _ in range(40):                                   # a few milliseconds of writes queued on A
        lib.sideaware_memcpy(p, ones.data_ptr(), n, 0, a.cuda_stream)
    lib.sideaware_free_auto(p, n, 0, a.cuda_stream)       # the host does not wait
    q = lib.sideaware_malloc_auto(n, 0, b.cuda_stream)
    assert q == p                                         # newest freed block of that size
    lib.sideaware_memcpy(q, twos.data_ptr(), n, 0, b.cuda_stream)
    torch.cuda.synchronize()
    lib.sideaware_memcpy(result.data_ptr(), q, n, 0, None)
    torch.cuda.synchronize()
    assert torch.equal(result, twos)                      # B's write came last
    after = sa.sideaware_alloc_stats()
    # the hand-over from A to B, and possibly one more when the region was first carved for A from
    # pages that an earlier test freed on the default stream
    assert before["stream_syncs"] + 1 <= after["stream_syncs"] <= before["stream_syncs"] + 2
    assert after["device_syncs"] == before["device_syncs"]          # the host never waited for the device
    lib.sideaware_free_auto(q, n, 0, b.cuda_stream)
    assert sa.sideaware_last_error() == ""


def test_multi_stream_churn_keeps_contents(sa):
    # Blocks are allocated and filled on one of four streams, then checked and freed on another
    # (ordered by an event, as a caller must), so freed pages keep moving between streams and
    # extents carry several of them.  A block handed out while an earlier owner's work was still
    # queued would show up as a wrong pattern.
    import time
    from l2_torch_alloc_amd import headers
    lib = sa.library()
    rng = random.Random(12)
    streams = [torch.cuda.Stream() for _ in range(4)]
    fill = lib.sideaware_create_kernel(headers.fill_header())
    staging = torch.empty(64 * MiB, dtype=torch.uint8, device="cuda")
    before = sa.sideaware_alloc_stats()
    live, checked = [], 0
    deadline = time.time() + 3.0
    while time.time() < deadline or live:
        if live and (time.time() >= deadline or len(live) > 100 or rng.random() < 0.45):
            ptr, n, si, val = live.pop(rng.randrange(len(live)))
            sj = rng.randrange(4)
            ev = torch.cuda.Event()
            ev.record(streams[si])
            streams[sj].wait_event(ev)
            with torch.cuda.stream(streams[sj]):
                lib.sideaware_memcpy(staging.data_ptr(), ptr, n, 0, streams[sj].cuda_stream)
                assert bool((staging[:n].view(torch.int32) == val).all()), "block %x of %d bytes" % (ptr, n)
            checked += 1
            lib.sideaware_free_auto(ptr, n, 0, streams[sj].cuda_stream)
        else:
            n = max(16, int(4096 * 2 ** (rng.random() * 14)) // 16 * 16)         # 4 KiB .. 64 MiB
            si = rng.randrange(4)
            ptr = lib.sideaware_malloc_auto(n, 0, streams[si].cuda_stream)
            assert ptr
            val = rng.randrange(1, 1 << 30)
            for _ in range(rng.choice([1, 1, 3])):                                # keep work queued behind the host
                lib.sideaware_elementwise(fill, n, ptr, 0, 0, 0, 0, 0, 0, 0, 0, val, 0, 0, 0, streams[si].cuda_stream)
            live.append((ptr, n, si, val))
    torch.cuda.synchronize()
    after = sa.sideaware_alloc_stats()
    assert checked > 1000
    assert after["stream_syncs"] > before["stream_syncs"] + 100      # hand-overs happened, ordered on the device
    assert after["failures"] == before["failures"] and sa.sideaware_last_error() == ""


def test_ready_made_ops_under_torch_compile(sa):
    # eager calls go straight to the op's implementation; while tracing, the same calls go through
    # torch.ops.sideaware.elementwise, which the tracer keeps as one opaque node
    from l2_torch_alloc_amd import ops
    x0 = torch.randn(2, 32, 4, 64, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16).cuda()
    freqs = ops.freqs_cis_table(64, 32, 10000.0).cuda()
    sb = torch.tensor([1.5, -0.25], dtype=torch.float32, device="cuda")
    eager = ops.scale_bias_bf16(ops.rope_forward_heads(x0.clone(), freqs), sb)

    @torch.compile(fullgraph=True)
    def step(x, freqs, sb):
        y = ops.rope_forward_heads(x, freqs)
        return ops.scale_bias_bf16(y, sb)

    out = step(x0.clone(), freqs, sb)
    torch.cuda.synchronize()
    assert torch.equal(out, eager)
    assert sa.sideaware_last_error() == ""


def test_first_use_of_a_ready_made_op_inside_torch_compile(sa):
    # no eager warm-up: the op's header is registered (a ctypes call) while the tracer runs, through
    # a function the tracer evaluates as a constant; shapes and dtypes no other test uses
    from l2_torch_alloc_amd import ops
    x0 = torch.randn(3, 24, 5, 48, generator=torch.Generator().manual_seed(9)).to(torch.float16).cuda()
    freqs = ops.freqs_cis_table(48, 24, 12345.0).cuda()
    assert not any(k[0] == "rope" and k[1][:4] == (24, 5, 0, 48) for k in ops._kernel_ids)

    @torch.compile(fullgraph=True)
    def step(x, freqs):
        return ops.rope_backward_heads(ops.rope_forward_heads(x, freqs), freqs)

    out = step(x0.clone(), freqs)
    torch.cuda.synchronize()
    want = ops.rope_backward_heads(ops.rope_forward_heads(x0.clone(), freqs), freqs)
    assert torch.equal(out, want)
    assert sa.sideaware_last_error() == ""
