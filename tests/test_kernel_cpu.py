"""Runs the shipped kernel template on the CPU, lane by lane, under AddressSanitizer.

The text comes out of the built library (``sideaware_kernel_source`` / ``sideaware_config_block``),
so what is checked is exactly what hipRTC compiles on the GPU box.  For each compile-time
configuration (index width, UNROLLED, traversal order) a small driver is built with the ROCm
clang as plain host C++ and fed many (grid, length, base offset, stripe, run) cases: the
workgroup -> tile map must visit every 16-byte vector exactly once, never touch a byte outside
the arrays, and do so for any grid size, which is the property the reference could not offer
(its map skips data unless exactly one block runs per SM, sideaware.cu:211-212).
"""
import ctypes
import os
import random
import subprocess

import pytest

from l2_torch_alloc_amd import build as sa_build

HERE = os.path.dirname(os.path.abspath(__file__))
NATIVE = os.path.join(HERE, "native")
CLANG = os.path.join(sa_build.rocm_root(), "lib", "llvm", "bin", "clang++")

INCREMENT_HEADER = """
typedef int o0;
typedef int i0;
struct unused {};
typedef unused o1, o2, o3, i1, i2, i3;
constexpr bool reverse_order = %(reverse)s;
constexpr bool input_evict[4] = {true, false, false, false};
%(unrolled)s
__device__ void elementwise_op(size_t element_idx, int sideband,
                               o0 &out0, o1 &out1, o2 &out2, o3 &out3,
                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {
    out0 = in0 + 1;
}
"""

MIXED_HEADER = """
typedef float o0;
typedef short o1;
typedef int   o2;
typedef short i0;
typedef float i1;
struct unused {};
typedef unused o3, i2, i3;
constexpr bool reverse_order = %(reverse)s;
constexpr bool input_evict[4] = {true, true, false, false};
%(unrolled)s
__device__ void elementwise_op(size_t element_idx, int sideband,
                               o0 &out0, o1 &out1, o2 &out2, o3 &out3,
                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {
    out0 = (float)in0 + in1;
    out1 = (short)(in1 * 10.0f + (float)sideband);
    out2 = (int)element_idx;
}
"""

NARROW_HEADER = """
typedef short o0;
typedef float i0;
struct unused {};
typedef unused o1, o2, o3, i1, i2, i3;
constexpr bool reverse_order = %(reverse)s;
constexpr bool input_evict[4] = {true, false, false, false};
%(unrolled)s
__device__ void elementwise_op(size_t element_idx, int sideband,
                               o0 &out0, o1 &out1, o2 &out2, o3 &out3,
                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {
    out0 = (short)in0 + 1;
}
"""

WIDEN_HEADER = """
typedef float o0;
typedef short i0;
struct unused {};
typedef unused o1, o2, o3, i1, i2, i3;
constexpr bool reverse_order = %(reverse)s;
constexpr bool input_evict[4] = {true, false, false, false};
%(unrolled)s
__device__ void elementwise_op(size_t element_idx, int sideband,
                               o0 &out0, o1 &out1, o2 &out2, o3 &out3,
                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {
    out0 = (float)in0 + 0.5f;
}
"""


@pytest.fixture(scope="module")
def lib():
    path = sa_build.build_library(force=False)
    L = ctypes.CDLL(path)
    L.sideaware_kernel_source.restype = ctypes.c_char_p
    L.sideaware_config_block.restype = ctypes.c_char_p
    L.sideaware_config_block.argtypes = [ctypes.c_int]
    L.sideaware_tune.argtypes = [ctypes.c_char_p, ctypes.c_longlong]
    return L


def build_driver(lib, tmp_path, case, variant, unrolled, reverse, header=None):
    config = lib.sideaware_config_block(variant).decode()
    template = lib.sideaware_kernel_source().decode()
    if header is None:
        header = {"INCREMENT": INCREMENT_HEADER, "MIXED": MIXED_HEADER, "NARROW": NARROW_HEADER, "WIDEN": WIDEN_HEADER}[case] % {
            "reverse": "true" if reverse else "false",
            "unrolled": "" if unrolled is None else "#define UNROLLED %d" % unrolled,
        }
    tu = "\n".join([
        '#include "%s"' % os.path.join(NATIVE, "kernel_cpu_prelude.h"),
        config, header, template,
        "#define SA_CASE_%s 1" % case,
        '#include "%s"' % os.path.join(NATIVE, "kernel_cpu_driver.h"),
    ])
    src = tmp_path / ("tu_%s_v%d_u%s_r%d_%x.cpp" % (case, variant, unrolled, reverse, hash(header) & 0xffffff))
    exe = str(src)[:-4]
    src.write_text(tu)
    cmd = [CLANG, "-x", "c++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined",
           "-fno-sanitize-recover=undefined", "-Wno-unused-value", str(src), "-o", exe]
    subprocess.run(cmd, check=True, capture_output=True, text=True)
    return exe


def cases_for(variant, unrolled, rng):
    tile = 256 * (unrolled or 4)
    lengths = {0, 1, 2, 15, 16, 255, 256, 257, tile - 1, tile, tile + 1, 2 * tile, 8 * tile, 8 * tile + 1,
               64 * tile - 1, 777, 3108 // 4}      # 777: the reference's (4, 777) fp32 case is 777 vectors
    lengths |= {rng.randrange(0, 70 * tile) for _ in range(40)}
    # every residue class of the tail for one tile count, sampled
    lengths |= {5 * tile + r for r in rng.sample(range(tile), 24)}
    grids = [0, 8, 16, 24, 56, 8 * 37, 2048]       # 0: one workgroup per tile
    offsets = [0, 16, 4096, 16384 + 32, 3 * 65536 + 4096 + 48, (2 << 20) - 16]
    stripes = [12, 14, 16, 18, 21, 24]          # log2 bytes: 4 KiB .. 16 MiB
    runs = [0, 1, 2, 3, 16, 1000]               # 0 = one contiguous block per workgroup
    out = []
    for n in sorted(lengths):
        for g in rng.sample(grids, 2):
            for off in rng.sample(offsets, 2):
                out.append((g, n, off, rng.choice(stripes), rng.choice(runs)))
    return out


CONFIGS = [
    # case, variant (0: 32-bit indices, 1: 64-bit), UNROLLED (None = template default), reverse_order
    ("INCREMENT", 0, None, False),
    ("INCREMENT", 1, None, False),
    ("INCREMENT", 0, 1, True),
    ("INCREMENT", 1, 2, True),
    ("INCREMENT", 1, 3, False),      # tile is not a power of two
    ("INCREMENT", 0, 8, False),      # tile larger than the smallest stripe
    ("INCREMENT", 0, 2, False),      # the built-in copy's setting
    ("MIXED", 0, None, False),
    ("MIXED", 1, 2, True),
    # variant bit 5: the sided ownership map (tiles of 4 KiB and of 8 KiB, both index widths, both orders)
    ("INCREMENT", 32, 1, False),
    ("INCREMENT", 33, 2, True),
    ("INCREMENT", 32, 2, False),
    ("INCREMENT", 33, 1, True),
    ("MIXED", 32, 1, False),         # o0 is wider than i0 but as wide as i1: the map follows o0
    ("INCREMENT", 32, 4, False),     # tiles of 16 KiB cannot be sided: the instantiation falls back to stripes
    ("NARROW", 0, None, False),      # i0 is wider than o0: stripes follow i0
    ("NARROW", 32, 1, False),        # ... and so does the sided map
    ("NARROW", 33, 2, True),
    ("WIDEN", 0, None, False),       # every input narrower than o0: stripes follow o0 ...
    ("WIDEN", 32, 1, False),         # ... the sided map follows i0, whose tiles are 2 KiB here
    ("WIDEN", 33, 4, True),          # and 8 KiB here (16 KiB of o0)
]


@pytest.mark.parametrize("case,variant,unrolled,reverse", CONFIGS)
def test_template_on_cpu(lib, tmp_path, case, variant, unrolled, reverse):
    if not os.path.exists(CLANG):
        pytest.skip("ROCm clang++ not found")
    exe = build_driver(lib, tmp_path, case, variant, unrolled, reverse)
    rng = random.Random(hash((case, variant, unrolled, reverse)) & 0xffff)
    cases = cases_for(variant, unrolled, rng)
    if case in ("MIXED", "NARROW", "WIDEN"):
        cases = [(g, n, off - off % 64, s, r) for (g, n, off, s, r) in cases]   # halved offsets stay 16 B-aligned
        lines = ["%d %d %d %d %d\n" % c for c in cases]
    else:
        # every case through the single-array entry point, and a fifth of them again cut into 2..8
        # segments that share one grid of the batched entry point
        lines = ["%d %d %d %d %d\n" % c for c in cases]
        lines += ["%d %d %d %d %d %d\n" % ((min(c[0], 56),) + c[1:] + (rng.choice([2, 3, 5, 8]),))
                  for c in rng.sample(cases, len(cases) // 5)]
    proc = subprocess.run([exe], input="".join(lines), capture_output=True, text=True, timeout=600,
                          env=dict(os.environ, ASAN_OPTIONS="detect_leaks=0"))
    assert proc.returncode == 0, proc.stdout[-3000:] + proc.stderr[-3000:]
    assert "cases=%d failed=0" % len(lines) in proc.stdout


ROPE_SHAPES = [
    # T, n_q, n_kv, head_dim, dtype, layout, backward-free forward only; variant
    (8, 3, 3, 8, "fp32", "qkv", 0),
    (16, 12, 12, 64, "fp32", "qkv", 1),
    (5, 4, 1, 16, "fp32", "qkv", 1),          # GQA head counts, T not a power of two
    (8, 32, 0, 128, "bf16", "heads", 0),
    (6, 8, 0, 128, "bf16", "heads", 1),
    (4, 4, 2, 32, "bf16", "qkv", 1),
    (8, 5, 0, 64, "fp16", "heads", 0),
    (4, 4, 2, 16, "fp16", "qkv", 1),
]


@pytest.mark.parametrize("T,n_q,n_kv,head_dim,dtype,layout,variant", ROPE_SHAPES)
def test_rope_headers_on_cpu(lib, tmp_path, T, n_q, n_kv, head_dim, dtype, layout, variant):
    if not os.path.exists(CLANG):
        pytest.skip("ROCm clang++ not found")
    from l2_torch_alloc_amd import headers
    header = headers.rope_header(T, n_q, n_kv, head_dim, dtype, layout).decode()
    exe = build_driver(lib, tmp_path, "ROPE", variant, None, False, header=header)
    heads = n_q + 2 * n_kv if layout == "qkv" else n_q
    pair_bytes = 8 if dtype == "fp32" else 4
    vecs_per_token = heads * (head_dim // 2) * pair_bytes // 16
    rng = random.Random(T * 131 + heads)
    cases = []
    for tokens in (1, T - 1, T, T + 1, 3 * T, 7 * T + 2):
        nv = tokens * vecs_per_token
        for grid in rng.sample([0, 8, 16, 56, 2048], 2):
            for off in (0, 16, 4096 + 32):
                cases.append((grid, nv, off, rng.choice([12, 14, 18, 22]), rng.choice([0, 1, 4])))
    cases.append((8, 3 * vecs_per_token + 1, 0, 14, 1))   # length that is not a whole number of tokens
    text = "".join("%d %d %d %d %d\n" % c for c in cases)
    proc = subprocess.run([exe], input=text, capture_output=True, text=True, timeout=600,
                          env=dict(os.environ, ASAN_OPTIONS="detect_leaks=0"))
    assert proc.returncode == 0, proc.stdout[-3000:] + proc.stderr[-3000:]
    assert "cases=%d failed=0" % len(cases) in proc.stdout
