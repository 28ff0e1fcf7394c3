"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle.

memcpy, fill and the mixed-width op are bit-exact.  fp32 RoPE is held to 1e-6 relative
(|got - want| <= 1e-6 * max(|want|, tiny)), and is expected to be bit-identical because neither
side fuses multiply and add; bf16 RoPE and scale+bias are held to 1 bf16 ulp, again expected
exact.  Full-size cases run at the shapes of the benchmark workloads; where the oracle would be
slow, size-independent properties take over (backward(forward(x)) == x, equality of two runs).
"""
import ctypes
import os

import numpy as np
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
MiB = 1 << 20


def bits(t: torch.Tensor) -> np.ndarray:
    """Host copy of a tensor's raw bytes as an unsigned integer array (NaN-safe comparisons)."""
    t = t.detach().contiguous().cpu()
    view = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[t.element_size()]
    return t.view(view).numpy().view({1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[t.element_size()])


def bf16_tensor(bits_u16: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(bits_u16.view(np.int16).copy()).view(torch.bfloat16)


def assert_no_library_error(sa):
    assert sa.sideaware_last_error() == "", sa.sideaware_last_error()


# --------------------------------------------------------------------------------------- start-up

def test_metadata(sa):
    info = sa.sideaware_info()
    lib = sa.library()
    print("sideaware metadata:", info, "xcds:", lib.sideaware_num_xcds(),
          "dealing verified:", lib.sideaware_xcd_dealing_verified())
    assert info["num_sms"] == torch.cuda.get_device_properties(0).multi_processor_count
    assert lib.sideaware_num_xcds() >= 1
    assert info["num_sms"] % lib.sideaware_num_xcds() == 0
    # the sides are the two halves of the device; the hash is what the start-up probe measured
    assert info["min"] >= 1 and info["hash"] == lib.sideaware_hash_mask() == lib.sideaware_side_address_mask()
    assert info["hash"] == 0 or info["hash"] & (1 << 13)
    table = sa.sideaware_torch_side_index().cpu().numpy()
    assert table.shape == (info["num_sms"],)
    side = table & 1
    counts = np.bincount(side, minlength=2)
    assert counts.sum() == info["num_sms"] and counts[0] == info["side0"] and counts[1] == info["side1"]
    assert info["min"] == min(info["side0"], info["side1"]) or lib.sideaware_num_xcds() == 1
    if lib.sideaware_num_xcds() == 8:
        assert info["side0"] == info["side1"] == info["num_sms"] // 2
    # ranks within each side count up from zero without gaps (the reference's table layout)
    for sd in range(2):
        ranks = np.sort(table[side == sd] >> 1)
        assert np.array_equal(ranks, np.arange(len(ranks)) & 0x7f)
    # the host copy the library returns a pointer to holds the same bytes
    host = (ctypes.c_ubyte * info["num_sms"]).from_address(sa.sideaware_cpu_side_index())
    assert np.array_equal(np.frombuffer(host, dtype=np.uint8), table)


# --------------------------------------------------------------------------------------- memcpy

@pytest.mark.parametrize("nbytes", [16, 256, 4096, 12432, 16384, 16400, 65536 + 4080, MiB, 8 * MiB,
                                    8 * MiB + 48, 64 * MiB, 256 * MiB])
def test_memcpy_bit_exact(sa, nbytes):
    g = torch.Generator().manual_seed(nbytes)
    src_host = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, generator=g)
    src = src_host.cuda()
    dst = torch.full((nbytes + 512,), 0xA5, dtype=torch.uint8, device="cuda")   # 256 guard bytes each side
    inner = dst[256:256 + nbytes]
    torch.ops.sideaware.memcpy(inner, src)
    torch.cuda.synchronize()
    assert_no_library_error(sa)
    out = dst.cpu()
    assert torch.equal(out[256:256 + nbytes], src_host)
    assert bool((out[:256] == 0xA5).all()) and bool((out[256 + nbytes:] == 0xA5).all())
    assert np.array_equal(O.memcpy(src_host.numpy()), out[256:256 + nbytes].numpy())


def test_memcpy_aligned_regions_take_the_fast_variant(sa):
    # two fresh 256 MiB tensors come straight from the large pool: 2 MiB-aligned, same stripe phase
    n = 256 * MiB
    src = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda")
    dst = torch.zeros_like(src)
    assert src.data_ptr() % (2 * MiB) == 0 and dst.data_ptr() % (2 * MiB) == 0
    torch.ops.sideaware.memcpy(dst, src)
    torch.cuda.synchronize()
    assert torch.equal(dst, src)
    assert_no_library_error(sa)


@pytest.mark.parametrize("dtype,shape,start", [
    (torch.float32, (4, 777), 0),            # 12,432 bytes: all tail (test.py:310)
    (torch.int16, (1000, 1000), 0),          # test.py:314
    (torch.float64, (1000, 1000), 0),        # test.py:315
    (torch.float32, (10000, 1000), 0),       # ~40 MB (test.py:316)
    (torch.float32, (10000, 1000), 3),       # a slice: base 12,000 bytes into the region
    (torch.bfloat16, (3, 5, 7, 64), 1),
])
def test_memcpy_shapes_and_dtypes_vs_copy_(sa, dtype, shape, start):
    n = int(np.prod(shape))
    src = torch.arange(n, device="cuda").to(dtype).reshape(shape)
    dst_ours = torch.zeros_like(src)
    dst_torch = torch.zeros_like(src)
    torch.ops.sideaware.memcpy(dst_ours[start:], src[start:])
    dst_torch[start:].copy_(src[start:])
    torch.cuda.synchronize()
    assert np.array_equal(bits(dst_ours), bits(dst_torch))
    assert_no_library_error(sa)


def test_memcpy_nan_payloads_survive(sa):
    pattern = torch.tensor([0x7FC00001, 0xFFC12345 - (1 << 32), 0x7F800001, 0], dtype=torch.int32).repeat(1024)
    src = pattern.cuda().view(torch.float32)
    dst = torch.zeros_like(src)
    torch.ops.sideaware.memcpy(dst, src)
    torch.cuda.synchronize()
    assert np.array_equal(bits(dst), bits(src))


def test_memcpy_between_the_cache_size_and_2_gib(sa):
    # 320 MiB + a tail: the all-streaming kernel class with 32-bit indices
    n = 320 * MiB + 4096 + 48
    src = torch.empty(n, dtype=torch.uint8, device="cuda")
    src.random_(0, 256)
    dst = torch.zeros_like(src)
    torch.ops.sideaware.memcpy(dst, src)
    torch.cuda.synchronize()
    assert torch.equal(dst, src)
    assert_no_library_error(sa)


def test_launches_replay_from_a_hip_graph(sa):
    # a launch allocates nothing and synchronises nothing, so it can be captured; the kernels are
    # compiled by a first eager call, outside the capture
    from l2_torch_alloc_amd import ops
    n = 8 * MiB + 4096
    src = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda")
    mid = torch.zeros_like(src)
    dst = torch.zeros_like(src)
    x = torch.randn(1, 64, 8, 128).to(torch.bfloat16).cuda()
    freqs = ops.freqs_cis_table(128, 64, 500000.0).cuda()
    x0 = x.clone()
    torch.ops.sideaware.memcpy(mid, src)
    ops.rope_forward_heads(x.clone(), freqs)
    torch.cuda.synchronize()
    eager = ops.rope_forward_heads(x0.clone(), freqs).clone()

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            torch.ops.sideaware.memcpy(mid, src)
            torch.ops.sideaware.memcpy(dst, mid)
            ops.rope_forward_heads(x, freqs)
    torch.cuda.current_stream().wait_stream(side)
    for trial in range(4):
        src.random_(0, 256)
        dst.zero_()
        x.copy_(x0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(dst, src), trial
        assert torch.equal(x, eager), trial
    assert_no_library_error(sa)


def test_memcpy_needs_64_bit_indices(sa):
    # 2 GiB + 64 KiB + 16 B: past the 32-bit path of the launcher (sideaware.cu:1387) and with a tail
    n = (2 << 30) + 65536 + 16
    src = torch.empty(n, dtype=torch.uint8, device="cuda")
    src.view(torch.int64)[: n // 8] = torch.arange(n // 8, device="cuda", dtype=torch.int64) * 0x9E3779B97F4A7C15
    dst = torch.zeros_like(src)
    torch.ops.sideaware.memcpy(dst, src)
    torch.cuda.synchronize()
    assert torch.equal(dst, src)
    assert_no_library_error(sa)


def test_memcpy_6gb_like_the_reference_script(sa):
    # (100000, 15000) fp32 = 6 GB (test.py:311)
    src = torch.arange(100000 * 15000, dtype=torch.float32, device="cuda").reshape(100000, 15000)
    dst = torch.zeros_like(src)
    torch.ops.sideaware.memcpy(dst, src)
    torch.cuda.synchronize()
    assert torch.equal(dst.view(torch.int32), src.view(torch.int32))


def test_memcpy_on_a_side_stream(sa):
    n = 32 * MiB
    src = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda")
    dst = torch.zeros_like(src)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        torch.ops.sideaware.memcpy(dst, src)
    stream.synchronize()
    assert torch.equal(dst, src)


def test_launch_knobs_do_not_change_results(sa):
    n = 24 * MiB + 4096 + 32
    src = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda")
    lib = sa.library()
    for groups, per_xcd in [(1, 0), (2, 1), (3, 5), (8, 0), (16, 31)]:
        dst = torch.zeros_like(src)
        lib.sideaware_elementwise(0, n, dst.data_ptr(), 0, 0, 0, src.data_ptr(), 0, 0, 0, 0, 0,
                                  groups, per_xcd, 0, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        assert torch.equal(dst, src), (groups, per_xcd)
    assert_no_library_error(sa)


def test_misuse_is_reported_not_fatal(sa):
    lib = sa.library()
    x = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    y = torch.ones(4096, dtype=torch.uint8, device="cuda")
    lib.sideaware_clear_error()
    lib.sideaware_memcpy(x.data_ptr() + 8, y.data_ptr(), 1024, 0, None)       # 8-byte aligned only
    assert "multiples of 16" in sa.sideaware_last_error()
    lib.sideaware_clear_error()
    lib.sideaware_memcpy(x.data_ptr(), y.data_ptr(), 1000, 0, None)           # length not a multiple of 16
    assert "multiples of 16" in sa.sideaware_last_error()
    lib.sideaware_clear_error()
    lib.sideaware_one_to_one(9999, 1024, x.data_ptr(), y.data_ptr(), 0, None)
    assert "never created" in sa.sideaware_last_error()
    bad = lib.sideaware_create_kernel(b"typedef int o0; this does not compile")
    lib.sideaware_clear_error()
    lib.sideaware_one_to_one(bad, 1024, x.data_ptr(), y.data_ptr(), 0, None)
    assert "failed to compile" in sa.sideaware_last_error()
    torch.cuda.synchronize()
    assert int(x.sum()) == 0                                                   # nothing ran
    lib.sideaware_clear_error()


# --------------------------------------------------------------------------------------- custom ops

MIXED_HEADER = b"""
#include <cuda_fp16.h>
#include <cuda_bf16.h>
typedef float o0;
typedef half o1;
typedef __nv_bfloat16 i0;
typedef float i1;
struct unused {};
typedef unused o2, o3, i2, i3;
__device__ void elementwise_op(size_t element_idx, int sideband,
                               o0 &out0, o1 &out1, o2 &out2, o3 &out3,
                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {
    out0 = (o0)((float)in0 + (float)in1);
    out1 = (o1)((float)in1 * 10.0f);
}
constexpr bool reverse_order = true;
constexpr bool input_evict[4] = {1,1,1,1};
"""


@pytest.mark.parametrize("n", [64, 1024 * 1024 + 64])
def test_two_in_two_out_mixed_widths(sa, n):
    # the reference's run-time-compile check (test.py:218-230): small integers, exact in bf16/fp16
    in0 = (torch.arange(n, device="cuda", dtype=torch.float32) % 64).to(torch.bfloat16)
    in1 = torch.ones(n, device="cuda", dtype=torch.float32) * 2
    out0 = torch.zeros(n, device="cuda", dtype=torch.float32)
    out1 = torch.zeros(n, device="cuda", dtype=torch.float16)
    kid = sa.sideaware_create_kernel(MIXED_HEADER)
    torch.ops.sideaware.elementwise(kid, out0, out1, None, None, in0, in1, None, None, None, 0, 0, 0)
    torch.cuda.synchronize()
    assert_no_library_error(sa)
    assert torch.equal(out0, in0.float() + in1)
    assert torch.equal(out1, (in1 * 10.0).half())


def test_reverse_order_with_persistent_grids(sa):
    # reverse_order walks each XCD's tiles from the end; with a fixed number of workgroups per CU the
    # grid is persistent and every workgroup loops.  Lengths with and without a partial last tile.
    lib = sa.library()
    kid = sa.sideaware_create_kernel(MIXED_HEADER)          # its header sets reverse_order = true
    stream = torch.cuda.current_stream().cuda_stream
    for n in (4096 * 37, 4096 * 37 + 52, 1000):
        in0 = (torch.arange(n, device="cuda", dtype=torch.float32) % 64).to(torch.bfloat16)
        in1 = torch.full((n,), 3.0, device="cuda", dtype=torch.float32)
        for groups, per_xcd in ((1, 1), (2, 3), (4, 0)):
            out0 = torch.zeros(n, device="cuda", dtype=torch.float32)
            out1 = torch.zeros(n, device="cuda", dtype=torch.float16)
            lib.sideaware_elementwise(kid, n * 4, out0.data_ptr(), out1.data_ptr(), 0, 0, in0.data_ptr(),
                                      in1.data_ptr(), 0, 0, 0, 0, groups, per_xcd, 0, stream)
            torch.cuda.synchronize()
            assert torch.equal(out0, in0.float() + in1), (n, groups, per_xcd)
            assert torch.equal(out1, (in1 * 10.0).half()), (n, groups, per_xcd)
    assert_no_library_error(sa)


def test_output_only_fill(sa):
    from l2_torch_alloc_amd import ops
    out = torch.zeros(3 * MiB // 4 + 4, dtype=torch.int32, device="cuda")
    ops.fill_int32(out, 0x5EEDBEEF)
    torch.cuda.synchronize()
    assert_no_library_error(sa)
    assert bool((out == 0x5EEDBEEF).all())


def test_scale_bias_bf16_vs_oracle_and_golden(sa):
    from l2_torch_alloc_amd import ops
    g = np.load(os.path.join(GOLDEN, "scale_bias_bf16.npz"))
    x = bf16_tensor(g["x"]).cuda()
    sb = torch.tensor([float(g["scale"]), float(g["bias"])], dtype=torch.float32, device="cuda")
    y = ops.scale_bias_bf16(x, sb)
    torch.cuda.synchronize()
    assert np.array_equal(bits(y), g["y"])
    # a larger seeded case against the oracle directly, other constants, same compiled kernel
    gen = torch.Generator().manual_seed(5)
    xh = torch.randn(5 * MiB + 8, generator=gen).to(torch.bfloat16)
    sb2 = torch.tensor([1.7, -0.3], dtype=torch.float32, device="cuda")
    y2 = ops.scale_bias_bf16(xh.cuda(), sb2)
    torch.cuda.synchronize()
    want = O.scale_bias_bf16(bits(xh), float(np.float32(1.7)), float(np.float32(-0.3)))
    assert O.bf16_ulp_distance(bits(y2), want).max() <= 1
    assert np.array_equal(bits(y2), want)
    assert_no_library_error(sa)


def test_mxfp8_quantize_vs_oracle(sa):
    # the vector_op + sideband op: bf16 -> E4M3 bytes + one E8M0 scale byte per 32 elements
    from l2_torch_alloc_amd import ops
    gen = torch.Generator().manual_seed(17)
    n = 32 * 40000 + 32 * 7                       # many tiles and a tail
    mag = torch.exp(torch.rand(n // 32, generator=gen) * 40 - 20).repeat_interleave(32)
    xh = (torch.randn(n, generator=gen) * mag).to(torch.bfloat16)
    xh[:32] = 0                                   # an all-zero block
    xh[32:64] = 1.0                               # a power-of-two block
    xh[64] = -1.9921875                           # saturates at -448 after scaling
    q, s = ops.mxfp8_quantize(xh.cuda())
    torch.cuda.synchronize()
    assert_no_library_error(sa)
    want_q, want_s = O.mxfp8_quantize(bits(xh))
    assert np.array_equal(s.cpu().numpy(), want_s)
    assert np.array_equal(q.cpu().numpy(), want_q)
    # The scale bytes leave through two routes (one 16-byte store per full wave; single bytes in the
    # last, partial wave, for a scale array off a 16-byte boundary, and for a launch that does not
    # pass the vector count): lengths around the wave size, a misaligned scale array with guard
    # bytes, and the raw entry point with sideband value 0.
    for blocks in (1, 15, 16, 17, 31, 33, 64 + 5, 1024 + 16):
        m = 32 * blocks
        x = xh[64:64 + m].clone().cuda()
        want_q, want_s = O.mxfp8_quantize(bits(xh[64:64 + m].clone()))
        for shift in (0, 1, 4):
            pad = torch.full((blocks + 64,), 0xEE, dtype=torch.uint8, device="cuda")
            scales = pad[16 + shift: 16 + shift + blocks]
            qq, ss = ops.mxfp8_quantize(x, scales=scales)
            torch.cuda.synchronize()
            assert np.array_equal(ss.cpu().numpy(), want_s), (blocks, shift)
            assert np.array_equal(qq.cpu().numpy(), want_q), (blocks, shift)
            assert bool((pad[:16 + shift] == 0xEE).all()) and bool((pad[16 + shift + blocks:] == 0xEE).all()), (blocks, shift)
    lib = sa.library()
    x = xh[:32 * 200].clone().cuda()
    want_q, want_s = O.mxfp8_quantize(bits(xh[:32 * 200].clone()))
    qq = torch.empty(32 * 200, dtype=torch.uint8, device="cuda")
    ss = torch.empty(200, dtype=torch.uint8, device="cuda")
    from l2_torch_alloc_amd import headers
    kid = sa.sideaware_create_kernel(headers.mxfp8_quantize_header())
    lib.sideaware_elementwise(kid, x.numel() * 2, qq.data_ptr(), 0, 0, 0, x.data_ptr(), 0, 0, 0, ss.data_ptr(), 0, 0, 0, 0,
                              torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert np.array_equal(ss.cpu().numpy(), want_s) and np.array_equal(qq.cpu().numpy(), want_q)
    # size-independent property at a large size: quantising the dequantised values changes nothing
    big = (torch.randn(64 * MiB // 2, generator=gen) * 3).to(torch.bfloat16).cuda()
    q1, s1 = ops.mxfp8_quantize(big)
    deq = (q1.view(torch.float8_e4m3fn).float() *
           torch.exp2(s1.float() - 127).repeat_interleave(32)).to(torch.bfloat16)
    q2, s2 = ops.mxfp8_quantize(deq)
    torch.cuda.synchronize()
    assert torch.equal(q1, q2) and torch.equal(s1, s2)


def test_mxfp8_dequantize_vs_oracle(sa):
    from l2_torch_alloc_amd import ops
    gen = torch.Generator().manual_seed(18)
    n = 32 * 30000 + 32 * 5
    mag = torch.exp(torch.rand(n // 32, generator=gen) * 40 - 20).repeat_interleave(32)
    xh = (torch.randn(n, generator=gen) * mag).to(torch.bfloat16)
    q_h, s_h = O.mxfp8_quantize(bits(xh))
    got = ops.mxfp8_dequantize(torch.from_numpy(q_h).cuda(), torch.from_numpy(s_h).cuda())
    torch.cuda.synchronize()
    assert_no_library_error(sa)
    want = O.mxfp8_dequantize(q_h, s_h)
    assert np.array_equal(bits(got), want)
    # an independent route to the same numbers: torch's own float8 decoding and power of two
    via_torch = (torch.from_numpy(q_h).view(torch.float8_e4m3fn).float() *
                 torch.exp2(torch.from_numpy(s_h).float() - 127).repeat_interleave(32)).to(torch.bfloat16)
    assert np.array_equal(bits(via_torch), want)
    # every E4M3 code except the two NaNs, under scale bytes from one end of E8M0 to the other
    # (results from bf16 subnormals up to infinity)
    codes = np.array([c for c in range(256) if c & 0x7f != 0x7f] + [0] * 2, dtype=np.uint8)      # 256 entries
    scale_bytes = np.array([0, 1, 9, 60, 127, 128, 200, 246, 254], dtype=np.uint8)
    q_all = np.tile(codes, len(scale_bytes))
    s_all = np.repeat(scale_bytes, len(codes) // 32)
    got = ops.mxfp8_dequantize(torch.from_numpy(q_all).cuda(), torch.from_numpy(s_all).cuda())
    torch.cuda.synchronize()
    want = O.mxfp8_dequantize(q_all, s_all)
    assert np.array_equal(bits(got), want)
    # and the pair is a projection: quantise(dequantise(q, s)) == (q, s) on the quantiser's own output
    q2, s2 = ops.mxfp8_quantize(ops.mxfp8_dequantize(torch.from_numpy(q_h).cuda(), torch.from_numpy(s_h).cuda()))
    torch.cuda.synchronize()
    assert np.array_equal(q2.cpu().numpy(), q_h) and np.array_equal(s2.cpu().numpy(), s_h)


# --------------------------------------------------------------------------------------- RoPE

def rel_err(got: np.ndarray, want: np.ndarray) -> float:
    return float(np.max(np.abs(got.astype(np.float64) - want) / np.maximum(np.abs(want), 1e-30)))


FP32_REL_TOL = 1e-6


@pytest.mark.parametrize("name", ["rope_fp32_qkv_tiny", "rope_fp32_qkv_gqa", "rope_fp32_qkv_scaled",
                                  "rope_fp32_heads_gpt2"])
def test_rope_fp32_golden(sa, name):
    from l2_torch_alloc_amd import ops
    g = np.load(os.path.join(GOLDEN, name + ".npz"))
    B, T, Nq, Nkv, HS = (int(v) for v in g["shape"])
    x = torch.from_numpy(g["x"]).cuda()
    freqs = torch.from_numpy(g["freqs"]).cuda()
    if "qkv" in name:
        y = ops.rope_forward_qkv(x.clone(), freqs, Nq, Nkv)
        dx = ops.rope_backward_qkv(y.clone(), freqs, Nq, Nkv)
    else:
        y = ops.rope_forward_heads(x.clone(), freqs)
        dx = ops.rope_backward_heads(y.clone(), freqs)
    torch.cuda.synchronize()
    assert_no_library_error(sa)
    assert np.array_equal(bits(y), g["y"].view(np.uint32))
    assert np.array_equal(bits(dx), g["dx"].view(np.uint32))


def test_rope_bf16_golden(sa):
    from l2_torch_alloc_amd import ops
    g = np.load(os.path.join(GOLDEN, "rope_bf16_heads_llama3.npz"))
    x = bf16_tensor(g["x"]).cuda()
    y = ops.rope_forward_heads(x, torch.from_numpy(g["freqs"]).cuda())
    torch.cuda.synchronize()
    assert O.bf16_ulp_distance(bits(y), g["y"]).max() <= 1
    assert np.array_equal(bits(y), g["y"])


def test_rope_fp32_gpt2_shape_vs_oracle(sa):
    # (B=4, T=1024, NH=12, HS=64) fp32, theta 1e4: in place and out of place
    from l2_torch_alloc_amd import ops
    B, T, NH, HS = 4, 1024, 12, 64
    gen = torch.Generator().manual_seed(1)
    xh = torch.randn(B, T, NH, HS, generator=gen)
    freqs_h = O.freqs_cis(HS, T, 10000.0)
    want = O.rope_forward_heads_f32(xh.numpy(), freqs_h)
    freqs = torch.from_numpy(freqs_h).cuda()
    x = xh.cuda()
    out = torch.empty_like(x)
    ops.rope_forward_heads(x, freqs, out=out)
    inplace = ops.rope_forward_heads(x.clone(), freqs)
    torch.cuda.synchronize()
    assert_no_library_error(sa)
    got = out.cpu().numpy()
    assert rel_err(got, want) <= FP32_REL_TOL
    assert O.validate_f32(got, want, 1e-5) == 0           # the reference harness's own rule
    assert np.array_equal(bits(out), want.view(np.uint32)), "expected bit-identical fp32"
    assert torch.equal(inplace, out)
    assert torch.equal(x.cpu(), xh)                       # out-of-place left the input alone


def test_rope_fp32_packed_qkv_reference_shape_vs_oracle(sa):
    # the reference benchmark's own tensor: (8, 1024, 3*32, 128) fp32, theta 1e4 with Llama-3.1
    # scaling (example_llmc_rope.cu:249-260); value heads must come through untouched
    from l2_torch_alloc_amd import ops
    B, T, NH, HS = 8, 1024, 32, 128
    gen = torch.Generator().manual_seed(8)
    xh = torch.randn(B, T, 3 * NH, HS, generator=gen)
    freqs_h = O.freqs_cis(HS, T, 10000.0, use_scaled=True)
    want = O.rope_forward_qkv_f32(xh.numpy(), freqs_h, NH, NH)
    x = xh.cuda()
    ops.rope_forward_qkv(x, torch.from_numpy(freqs_h).cuda(), NH, NH)
    torch.cuda.synchronize()
    got = x.cpu().numpy()
    assert rel_err(got, want) <= FP32_REL_TOL
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(got[:, :, 2 * NH:].view(np.uint32), xh.numpy()[:, :, 2 * NH:].view(np.uint32))
    # backward brings it back (conjugate rotation), to rounding
    ops.rope_backward_qkv(x, torch.from_numpy(freqs_h).cuda(), NH, NH)
    torch.cuda.synchronize()
    np.testing.assert_allclose(x.cpu().numpy(), xh.numpy(), atol=2e-6, rtol=2e-6)
    want_back = O.rope_backward_qkv_f32(want, freqs_h, NH, NH)
    assert np.array_equal(bits(x), want_back.view(np.uint32))


def test_rope_out_of_place_qkv_carries_value_heads(sa):
    from l2_torch_alloc_amd import ops
    B, T, Nq, Nkv, HS = 2, 16, 4, 2, 64
    xh = torch.randn(B, T, Nq + 2 * Nkv, HS, generator=torch.Generator().manual_seed(3))
    freqs_h = O.freqs_cis(HS, T, 500000.0)
    out = torch.full_like(xh, float("nan")).cuda()
    ops.rope_forward_qkv(xh.cuda(), torch.from_numpy(freqs_h).cuda(), Nq, Nkv, out=out)
    torch.cuda.synchronize()
    want = O.rope_forward_qkv_f32(xh.numpy(), freqs_h, Nq, Nkv)
    assert np.array_equal(bits(out), want.view(np.uint32))


def test_rope_bf16_llama3_full_size_vs_oracle(sa):
    # q (8, 4096, 32, 128) and k (8, 4096, 8, 128) bf16 in place, theta 5e5: the benchmark workload
    from l2_torch_alloc_amd import ops
    B, T, HS = 8, 4096, 128
    freqs_h = O.freqs_cis(HS, T, 500000.0)
    freqs = torch.from_numpy(freqs_h).cuda()
    gen = torch.Generator().manual_seed(2)
    for heads in (32, 8):
        xh = torch.randn(B, T, heads, HS, generator=gen).to(torch.bfloat16)
        x = xh.cuda()
        assert x.data_ptr() % (2 * MiB) == 0
        ops.rope_forward_heads(x, freqs)
        torch.cuda.synchronize()
        assert_no_library_error(sa)
        want = O.rope_forward_heads_bf16(bits(xh), freqs_h)
        got = bits(x)
        dist = O.bf16_ulp_distance(got, want)
        assert dist.max() <= 1, "more than 1 bf16 ulp from the fp32 oracle"
        assert np.array_equal(got, want), "expected bit-identical bf16 (%d differ)" % int((dist > 0).sum())
        del x, xh, want, got, dist


def test_rope_bf16_packed_gqa_vs_oracle(sa):
    # packed QKV with grouped heads in bf16: oracle = rotate the q|k slice as heads, keep v bits
    from l2_torch_alloc_amd import ops
    B, T, Nq, Nkv, HS = 2, 512, 32, 8, 128
    xh = torch.randn(B, T, Nq + 2 * Nkv, HS, generator=torch.Generator().manual_seed(9)).to(torch.bfloat16)
    freqs_h = O.freqs_cis(HS, T, 500000.0)
    x = xh.cuda()
    ops.rope_forward_qkv(x, torch.from_numpy(freqs_h).cuda(), Nq, Nkv)
    torch.cuda.synchronize()
    xb = bits(xh)
    want = xb.copy()
    want[:, :, :Nq + Nkv] = O.rope_forward_heads_bf16(np.ascontiguousarray(xb[:, :, :Nq + Nkv]), freqs_h)
    assert np.array_equal(bits(x), want)


def _oracle_rope(x_f32, freqs, layout, n_q, n_kv, backward):
    if layout == "qkv":
        fn = O.rope_backward_qkv_f32 if backward else O.rope_forward_qkv_f32
        return fn(x_f32, freqs, n_q, n_kv)
    fn = O.rope_backward_heads_f32 if backward else O.rope_forward_heads_f32
    return fn(x_f32, freqs)


def _random_rope_cases(count, seed):
    import random
    rng = random.Random(seed)
    cases = []
    while len(cases) < count:
        dtype = rng.choice(["fp32", "bf16", "fp16"])
        layout = rng.choice(["qkv", "heads"])
        head_dim = rng.choice([4, 8, 12, 64, 96, 128] if dtype == "fp32" else [8, 16, 32, 64, 128, 256])
        n_q = rng.randint(1, 8)
        n_kv = rng.randint(1, n_q) if layout == "qkv" else 0
        cases.append(dict(dtype=dtype, layout=layout, head_dim=head_dim, n_q=n_q, n_kv=n_kv,
                          B=rng.randint(1, 3), T=rng.choice([1, 2, 7, 33, 64, 100, 257]),
                          backward=rng.random() < 0.4, in_place=rng.random() < 0.5,
                          theta=rng.choice([10000.0, 500000.0]), scaled=rng.random() < 0.3,
                          seed=1000 + len(cases)))
    return cases


@pytest.mark.parametrize("case", _random_rope_cases(24, seed=20), ids=lambda c: "%s-%s-d%d-q%d-kv%d-B%d-T%d%s%s" % (
    c["dtype"], c["layout"], c["head_dim"], c["n_q"], c["n_kv"], c["B"], c["T"],
    "-bwd" if c["backward"] else "", "-inplace" if c["in_place"] else ""))
def test_rope_random_shapes_vs_oracle(sa, case):
    # Seeded random shapes, ragged against every tile size: head counts that are not powers of two,
    # T = 1, head_dim down to one vector per head, grouped k/v heads, forward and backward, in place
    # and out of place, all three storage types.  Bit for bit against the oracle (bf16 and fp16: the
    # oracle's fp32 arithmetic on the widened inputs, narrowed round-to-nearest-even).
    from l2_torch_alloc_amd import ops
    c = case
    heads = c["n_q"] + 2 * c["n_kv"] if c["layout"] == "qkv" else c["n_q"]
    gen = torch.Generator().manual_seed(c["seed"])
    xh = torch.randn(c["B"], c["T"], heads, c["head_dim"], generator=gen)
    if c["dtype"] == "bf16":
        xh = xh.to(torch.bfloat16)
    elif c["dtype"] == "fp16":
        xh = xh.to(torch.float16)
    freqs_h = O.freqs_cis(c["head_dim"], c["T"], c["theta"], c["scaled"])
    want = _oracle_rope(xh.float().numpy(), freqs_h, c["layout"], c["n_q"], c["n_kv"], c["backward"])
    x = xh.cuda()
    freqs = torch.from_numpy(freqs_h).cuda()
    out = None if c["in_place"] else torch.full_like(x, 7.0)
    fn = {("qkv", False): ops.rope_forward_qkv, ("qkv", True): ops.rope_backward_qkv,
          ("heads", False): ops.rope_forward_heads, ("heads", True): ops.rope_backward_heads}[(c["layout"], c["backward"])]
    got = fn(x, freqs, c["n_q"], c["n_kv"], out=out) if c["layout"] == "qkv" else fn(x, freqs, out=out)
    torch.cuda.synchronize()
    rotated = c["n_q"] + c["n_kv"] if c["layout"] == "qkv" else heads
    got_h = got.cpu()
    if c["dtype"] == "bf16":
        assert np.array_equal(bits(got_h[:, :, :rotated]), O.f32_to_bf16(want[:, :, :rotated]))
    elif c["dtype"] == "fp16":
        # IEEE round-to-nearest-even narrowing: numpy's float32 -> float16 conversion
        assert np.array_equal(bits(got_h[:, :, :rotated]), want[:, :, :rotated].astype(np.float16).view(np.uint16))
    else:
        assert np.array_equal(bits(got_h[:, :, :rotated]), want[:, :, :rotated].view(np.uint32))
    if rotated < heads:
        # value heads: untouched in place, carried over bit for bit out of place (as the oracle does)
        assert np.array_equal(bits(got_h[:, :, rotated:]), bits(xh[:, :, rotated:]))
    if not c["in_place"]:
        assert torch.equal(x.cpu(), xh)                     # the input is left alone
    assert_no_library_error(sa)


def test_host_threads_compile_and_launch_concurrently(sa):
    # The reference has no locking at all; here the registry and the compile cache are guarded.
    # Six host threads each register an op of their own (new text: a fresh compile), launch it on a
    # stream of their own next to a copy, and check the result.
    import threading
    from l2_torch_alloc_amd import headers
    lib = sa.library()
    n = 3 * MiB + 48
    errors = []

    def worker(tid):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                src = torch.full((n // 4,), tid + 1, dtype=torch.int32, device="cuda")
                dst = torch.zeros_like(src)
                filled = torch.zeros_like(src)
            text = headers.fill_header().replace(b"sideaware_fill_int32", b"sideaware_fill_thread%d" % tid)
            text = text.replace(b"out0 = sideband;", b"out0 = sideband + %d;" % (100 * tid))
            kid = lib.sideaware_create_kernel(text)
            assert kid > 0
            for _ in range(20):
                lib.sideaware_memcpy(dst.data_ptr(), src.data_ptr(), n, 0, stream.cuda_stream)
                lib.sideaware_elementwise(kid, n, filled.data_ptr(), 0, 0, 0, 0, 0, 0, 0, 0, 5, 0, 0, 0,
                                          stream.cuda_stream)
            stream.synchronize()
            assert torch.equal(dst, src), "copy on thread %d" % tid
            assert bool((filled == 5 + 100 * tid).all()), "fill on thread %d" % tid
        except Exception as e:      # reported by the main thread
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(6)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    assert_no_library_error(sa)


def test_rope_bf16_2gib_tensor_uses_64_bit_indices_and_matches_its_slices(sa):
    # (64, 4096, 32, 128) bf16 is exactly 2 GiB: the 64-bit index instantiation, all-streaming
    # class.  RoPE treats batch rows independently, so the result must equal, bit for bit, what
    # the 32-bit instantiation gives for each (8, 4096, 32, 128) slice on its own; one slice is
    # also held against the oracle.
    from l2_torch_alloc_amd import ops
    B, T, NH, HS = 64, 4096, 32, 128
    freqs_h = O.freqs_cis(HS, T, 500000.0)
    freqs = torch.from_numpy(freqs_h).cuda()
    x = torch.empty(B, T, NH, HS, dtype=torch.bfloat16, device="cuda")
    x.view(torch.int16).copy_(((torch.arange(x.numel(), device="cuda", dtype=torch.int64) * 2654435761) >> 7)
                              .to(torch.int16).view(B, T, NH, HS))
    x.view(torch.int16).bitwise_and_(0x3fff)               # finite, positive bf16 patterns below 2.0
    assert x.numel() * 2 == 2 << 30
    whole = x.clone()
    ops.rope_forward_heads(whole, freqs)
    for b0 in range(0, B, 8):
        part = x[b0:b0 + 8].clone()
        ops.rope_forward_heads(part, freqs)
        assert torch.equal(whole[b0:b0 + 8].view(torch.int16), part.view(torch.int16)), "slice at batch %d" % b0
    torch.cuda.synchronize()
    one = x[40:41].cpu()
    want = O.rope_forward_heads_bf16(bits(one), freqs_h)
    assert np.array_equal(bits(whole[40:41]), want)
    assert_no_library_error(sa)


def test_precompiled_kernel_with_default_groups(sa):
    # sideaware_create_kernel_advanced (sideaware.cu:1421-1458): precompile builds every
    # instantiation up front, default_num_groups makes a persistent grid the kernel's default
    import time
    from l2_torch_alloc_amd import headers
    lib = sa.library()
    text = headers.scale_bias_bf16_header().replace(b"sideaware_scale_bias_bf16", b"sideaware_scale_bias_precompiled")
    assert b"sideaware_scale_bias_precompiled" in text
    kid = lib.sideaware_create_kernel_advanced(text, True, 2)
    assert kid > 0 and lib.sideaware_create_kernel_advanced(text, False, 0) == kid
    info = (ctypes.c_int * 4)()
    assert lib.sideaware_kernel_info(kid, 0, info) == 0 and info[3] == 2      # default workgroups per CU
    n = 3 * MiB + 24
    xh = torch.randn(n, generator=torch.Generator().manual_seed(11)).to(torch.bfloat16)
    x = xh.cuda()
    y = torch.empty_like(x)
    sb = torch.tensor([0.5, 3.0], dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    lib.sideaware_elementwise(kid, 2 * n, y.data_ptr(), 0, 0, 0, x.data_ptr(), 0, 0, 0, sb.data_ptr(), 0, 0, 0, 0, stream)
    lib.sideaware_elementwise(kid, 2 * n, x.data_ptr(), 0, 0, 0, x.data_ptr(), 0, 0, 0, sb.data_ptr(), 0, 0, 0, 0, stream)
    torch.cuda.synchronize()
    assert time.perf_counter() - t0 < 0.05                  # out of place and in place: nothing left to compile
    want = O.scale_bias_bf16(bits(xh), 0.5, 3.0)
    assert np.array_equal(bits(y), want) and np.array_equal(bits(x), want)
    assert_no_library_error(sa)


INPUT_ONLY_SUM = b"""
#define KERNEL_NAME sideaware_test_input_only_sum
typedef int i0;
struct unused {};
typedef unused o0, o1, o2, o3, i1, i2, i3;
constexpr bool reverse_order = false;
constexpr bool input_evict[4] = {true, false, false, false};
__device__ void elementwise_op(size_t element_idx, int sideband, o0 &out0, o1 &out1, o2 &out2, o3 &out3,
                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {}
#define CUSTOM_VECTOR_OP
__device__ __forceinline__ void vector_op(size_type vec_idx, int vec_size, o0 *out0, o1 *out1, o2 *out2, o3 *out3,
                                          const i0 *in0, const i1 *in1, const i2 *in2, const i3 *in3,
                                          int* sideband_memory, int sideband_value) {
    atomicAdd(sideband_memory, (in0[0] + in0[1] + in0[2] + in0[3]) * sideband_value);
    atomicAdd(sideband_memory + 1, 1);
}
"""


@pytest.mark.parametrize("n_ints", [4, 1024 + 4, 5 * MiB // 4 + 12, 300 * MiB // 4])
def test_input_only_op_with_sideband_result(sa, n_ints):
    # No output array at all: every vector of the input is visited exactly once (the vector count
    # and a weighted sum arrive through the sideband pointer), for a tail-only array, tiles plus a
    # tail, and a size in the all-streaming class.
    lib = sa.library()
    kid = lib.sideaware_create_kernel(INPUT_ONLY_SUM)
    x = torch.randint(-1000, 1000, (n_ints,), dtype=torch.int32, device="cuda")
    acc = torch.zeros(4, dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    lib.sideaware_elementwise(kid, 4 * n_ints, 0, 0, 0, 0, x.data_ptr(), 0, 0, 0, acc.data_ptr(), 3, 0, 0, 0, stream)
    torch.cuda.synchronize()
    assert_no_library_error(sa)
    assert int(acc[1]) == n_ints // 4
    want = (3 * int(x.sum(dtype=torch.int64))) & 0xffffffff
    assert (int(acc[0]) & 0xffffffff) == want


NARROW_HEADER = """
typedef %(out)s o0;
typedef %(inp)s i0;
struct unused {};
typedef unused o1, o2, o3, i1, i2, i3;
__device__ void elementwise_op(size_t element_idx, int sideband,
                               o0 &out0, o1 &out1, o2 &out2, o3 &out3,
                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {
    out0 = (o0)(in0 + (i0)sideband);
}
constexpr bool reverse_order = false;
constexpr bool input_evict[4] = {1,0,0,0};
"""


@pytest.mark.parametrize("inp,out,tin,tout,per_lane", [
    ("double", "unsigned char", torch.float64, torch.uint8, 2),     # 2 elements per lane: 2-byte stores
    ("double", "short", torch.float64, torch.int16, 4),             # 4-byte stores
    ("float", "unsigned char", torch.float32, torch.uint8, 4),      # 4-byte stores
    ("float", "short", torch.float32, torch.int16, 8),              # 8-byte stores
    ("short", "double", torch.int16, torch.float64, 64),            # four 16-byte stores per lane
])
def test_outputs_narrower_and_wider_than_the_input(sa, inp, out, tin, tout, per_lane):
    # every store width of the template: 2, 4, 8 and several times 16 bytes per lane, in both
    # cache classes, with a partial last tile and guard elements behind the output
    lib = sa.library()
    stream = torch.cuda.current_stream().cuda_stream
    kid = sa.sideaware_create_kernel((NARROW_HEADER % {"inp": inp, "out": out}).encode())
    wide_bytes = max(torch.empty(0, dtype=tin).element_size(), torch.empty(0, dtype=tout).element_size())
    for n in (16 // wide_bytes * 5, 4096 * 3 + 16 // wide_bytes * 7, (300 << 20) // wide_bytes):
        x = (torch.arange(n, dtype=torch.int64, device="cuda") % 97).to(tin)
        # the output on a 64-byte boundary (write-through stores) and 16 bytes past one (the
        # instantiation with the compiler's stores)
        for shift in (0, 16 // torch.empty(0, dtype=tout).element_size()):
            y = torch.full((n + 64 + shift,), 7, dtype=tout, device="cuda")
            out_view = y[shift:]
            lib.sideaware_elementwise(kid, n * wide_bytes, out_view.data_ptr(), 0, 0, 0, x.data_ptr(), 0, 0, 0, 0, 3, 0, 0, 0,
                                      stream)
            torch.cuda.synchronize()
            assert_no_library_error(sa)
            assert torch.equal(out_view[:n], (x + 3).to(tout)), (inp, out, n, shift)
            assert bool((out_view[n:] == 7).all()) and bool((y[:shift] == 7).all()), (inp, out, n, shift)
    del per_lane


FOUR_BY_FOUR_HEADER = b"""
typedef float o0; typedef short o1; typedef double o2; typedef unsigned char o3;
typedef float i0; typedef int i1; typedef short i2; typedef unsigned char i3;
__device__ void elementwise_op(size_t element_idx, int sideband,
                               o0 &out0, o1 &out1, o2 &out2, o3 &out3,
                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {
    out0 = in0 + (float)in1;
    out1 = (short)(in2 + in3);
    out2 = (double)in0 * 2.0 + (double)sideband;
    out3 = (unsigned char)(in3 ^ (unsigned char)(element_idx & 0xff));
}
constexpr bool reverse_order = false;
constexpr bool input_evict[4] = {1,0,1,0};
"""


@pytest.mark.parametrize("n", [4, 1024 * 7 + 12, 5 * (1 << 20)])
def test_four_inputs_and_four_outputs_of_four_widths(sa, n):
    # the widest arrays (float in0, double out2 is wider still) set the vector: 16 bytes of the
    # wider of (i0, o0), so 4 elements per lane; out2 then takes 32 bytes per lane, out3 four
    kid = sa.sideaware_create_kernel(FOUR_BY_FOUR_HEADER)
    g = torch.Generator().manual_seed(n)
    in0 = torch.randint(-1000, 1000, (n,), generator=g).float().cuda()
    in1 = torch.randint(-1000, 1000, (n,), generator=g, dtype=torch.int32).cuda()
    in2 = torch.randint(-1000, 1000, (n,), generator=g, dtype=torch.int16).cuda()
    in3 = torch.randint(0, 200, (n,), generator=g, dtype=torch.uint8).cuda()
    out0 = torch.zeros(n, dtype=torch.float32, device="cuda")
    out1 = torch.zeros(n, dtype=torch.int16, device="cuda")
    out2 = torch.zeros(n, dtype=torch.float64, device="cuda")
    out3 = torch.zeros(n, dtype=torch.uint8, device="cuda")
    torch.ops.sideaware.elementwise(kid, out0, out1, out2, out3, in0, in1, in2, in3, None, 5, 0, 0)
    torch.cuda.synchronize()
    assert_no_library_error(sa)
    idx = (torch.arange(n, device="cuda") & 0xff).to(torch.uint8)
    assert torch.equal(out0, in0 + in1.float())
    assert torch.equal(out1, in2 + in3.to(torch.int16))
    assert torch.equal(out2, in0.double() * 2.0 + 5.0)
    assert torch.equal(out3, in3 ^ idx)
