"""The C-ABI boundary without a GPU: the library loads, exports every symbol that
include/sideaware.h declares (and binds with the ctypes signatures the reference's scripts use,
test.py:18-39 / example_wrapper.py:53-80), the header registry dedups, and every shipped op
header compiles for gfx950 in both index variants.  No compute call is made.
"""
import ctypes
import os
import re
import subprocess

import pytest

from l2_torch_alloc_amd import build as sa_build
from l2_torch_alloc_amd import headers, wrapper

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# The 26 entry points of the reference's extern "C" block (sideaware.cu:1278-1524).
REFERENCE_SYMBOLS = [
    "sideaware_malloc_async", "sideaware_free_async", "sideaware_malloc", "sideaware_free",
    "sideaware_release_unused", "sideaware_malloc_auto", "sideaware_free_auto",
    "sideaware_elementwise", "sideaware_one_to_one", "sideaware_memcpy",
    "sideaware_create_kernel_advanced", "sideaware_create_kernel",
    "sideaware_compression", "sideaware_alloc_threshold", "sideaware_prealloc_config",
    "sideaware_free_mapped_thresholds", "sideaware_write_sass",
    "sideaware_fill_side_index", "sideaware_gpu_side_index", "sideaware_cpu_side_index",
    "sideaware_sm_side_summary", "sideaware_num_sms", "sideaware_num_sm_side0",
    "sideaware_num_sm_side1", "sideaware_min_sm_per_side", "sideaware_hash_mask",
]


@pytest.fixture(scope="module")
def lib():
    return wrapper.bind(sa_build.build_library(force=False))


def declared_in_header():
    text = open(os.path.join(ROOT, "include", "sideaware.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sideaware_[a-z0-9_]+)\s*\(", text)))


def exported_by_library():
    out = subprocess.run(["nm", "-D", "--defined-only", sa_build.LIB_PATH], check=True,
                         capture_output=True, text=True).stdout
    return sorted(l.split()[-1] for l in out.splitlines() if " T " in l and "sideaware_" in l)


def test_every_declared_symbol_is_exported_and_nothing_else(lib):
    declared, exported = declared_in_header(), exported_by_library()
    assert declared == exported
    assert sorted(wrapper.EXPORTED_SYMBOLS) == declared
    missing = [s for s in REFERENCE_SYMBOLS if s not in exported]
    assert not missing, "reference entry points missing: %s" % missing


def test_reference_ctypes_signatures_bind(lib):
    # The declarations the reference's scripts make (test.py:18-39).  Binding a wrong arity is not
    # detectable through ctypes, so this only proves the names resolve and are callable objects;
    # the widths are pinned by include/sideaware.h, which the library is compiled against.
    L = ctypes.CDLL(sa_build.LIB_PATH)
    L.sideaware_create_kernel.argtypes = [ctypes.c_char_p]
    L.sideaware_create_kernel.restype = ctypes.c_int
    L.sideaware_sm_side_summary.restype = ctypes.POINTER(ctypes.c_int * 5)
    L.sideaware_memcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p]
    L.sideaware_elementwise.argtypes = [ctypes.c_int, ctypes.c_size_t] + [ctypes.c_void_p] * 10 + \
        [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    # with a pointer-sized sideband_value, as the reference declares it
    assert callable(L.sideaware_elementwise)


def test_header_registry_dedups_without_a_device(lib):
    assert lib.sideaware_create_kernel(None) == 0
    assert lib.sideaware_create_kernel(b"") == 0
    a = lib.sideaware_create_kernel(headers.fill_header())
    b = lib.sideaware_create_kernel(headers.scale_bias_bf16_header())
    assert a >= 1 and b == a + 1
    assert lib.sideaware_create_kernel(headers.fill_header()) == a
    assert lib.sideaware_create_kernel_advanced(headers.scale_bias_bf16_header(), False, 3) == b


def test_zero_byte_and_null_calls_return_before_touching_a_device(lib):
    lib.sideaware_clear_error()
    lib.sideaware_memcpy(0, 0, 0, 0, None)
    lib.sideaware_memcpy(0, 0, 4096, 0, None)          # both pointers null
    lib.sideaware_free_auto(None, 0, 0, None)
    lib.sideaware_elementwise_batch(0, 0, None, 0, None)
    from l2_torch_alloc_amd import ops
    empty = (ops._Segment * 3)()                       # three segments, none with anything to do
    empty[1].num_bytes = 4096                          # bytes but no pointers
    lib.sideaware_elementwise_batch(0, 3, empty, 0, None)
    assert lib.sideaware_last_error() == b""


def test_tuning_knobs(lib):
    assert lib.sideaware_tune(b"no_such_knob", 1) != 0
    assert lib.sideaware_tune(b"stripe_bytes", 12345) != 0        # not a power of two
    old = lib.sideaware_tune_get(b"stripe_bytes")
    assert lib.sideaware_tune(b"stripe_bytes", 65536) == 0
    assert lib.sideaware_tune_get(b"stripe_bytes") == 65536
    assert lib.sideaware_tune(b"stripe_bytes", old) == 0
    assert lib.sideaware_tune(b"slot_run", 0) == 0 and lib.sideaware_tune_get(b"slot_run") == 0
    assert lib.sideaware_tune(b"slot_run", 1) == 0
    assert b"using size_type = long long" in lib.sideaware_config_block(1)
    assert b"using size_type = int;" in lib.sideaware_config_block(0)
    assert b"#define SA_BEYOND_CACHE 0" in lib.sideaware_config_block(1)
    assert b"#define SA_BEYOND_CACHE 1" in lib.sideaware_config_block(2)
    old_nt = lib.sideaware_tune_get(b"nt_store")
    assert lib.sideaware_tune(b"nt_store", 0) == 0
    assert b"#define SA_NT_STORE 0" in lib.sideaware_config_block(0)
    assert lib.sideaware_tune(b"nt_store", old_nt) == 0


def compile_ok(lib, header, variant):
    log = ctypes.create_string_buffer(1 << 16)
    rc = lib.sideaware_compile_check(header, variant, log, len(log))
    return rc, log.value.decode()


SHIPPED_HEADERS = {
    "builtin_copy": None,
    "copy": headers.memcpy_header(),
    "fill": headers.fill_header(),
    "scale_bias_bf16": headers.scale_bias_bf16_header(),
    "mxfp8_quantize": headers.mxfp8_quantize_header(),
    "mxfp8_dequantize": headers.mxfp8_dequantize_header(),
    "rope_fp32_qkv_gpt2": headers.rope_header(1024, 12, 12, 64, "fp32", "qkv"),
    "rope_fp32_heads_gpt2": headers.rope_header(1024, 12, 0, 64, "fp32", "heads"),
    "rope_fp32_qkv_ref": headers.rope_header(1024, 32, 32, 128, "fp32", "qkv"),
    "rope_bf16_q_llama3": headers.rope_header(4096, 32, 0, 128, "bf16", "heads"),
    "rope_bf16_k_llama3": headers.rope_header(4096, 8, 0, 128, "bf16", "heads"),
    "rope_bf16_qkv_gqa": headers.rope_header(4096, 32, 8, 128, "bf16", "qkv"),
    "rope_fp32_backward": headers.rope_header(1024, 12, 12, 64, "fp32", "qkv", backward=True),
    "rope_fp16_q": headers.rope_header(2048, 16, 0, 64, "fp16", "heads"),
}


@pytest.mark.parametrize("name", sorted(SHIPPED_HEADERS))
@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4])
def test_shipped_headers_compile_for_gfx950(lib, name, variant):
    rc, log = compile_ok(lib, SHIPPED_HEADERS[name], variant)
    assert rc == 0, log
    assert "warning" not in log, log


# An op header in the reference's own dialect: CUDA header names, CUDA's bf16 type name, `half`,
# mixed element widths, reverse order (the shape of test.py:191-216, written afresh).
CUDA_DIALECT_HEADER = b"""
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
    out0 = (o0)((float)in0 - (float)in1);
    out1 = (o1)((float)in1 * 3.0f);
}
constexpr bool reverse_order = true;
constexpr bool input_evict[4] = {1,1,1,1};
"""


@pytest.mark.parametrize("variant", [0, 3])
def test_cuda_dialect_header_compiles(lib, variant):
    rc, log = compile_ok(lib, CUDA_DIALECT_HEADER, variant)
    assert rc == 0, log


def test_broken_header_reports_instead_of_aborting(lib):
    rc, log = compile_ok(lib, b"typedef int o0; this is not C++", 0)
    assert rc != 0 and "error" in log


def test_header_may_include_a_file_relative_to_the_working_directory(lib, tmp_path, monkeypatch):
    # example_llmc_rope.cu:138 registers the one-line header `#include "kernel_rope.cuh"` and relies
    # on the compiler finding the file in the process's working directory
    (tmp_path / "my_rope_op.h").write_bytes(headers.rope_header(1024, 32, 32, 128, "fp32", "qkv"))
    monkeypatch.chdir(tmp_path)
    rc, log = compile_ok(lib, b'#include "my_rope_op.h"\n', 0)
    assert rc == 0, log
    # the file's content is read at every compile, never served from the on-disk cache: a changed
    # file must not keep compiling as the old one
    (tmp_path / "my_rope_op.h").write_bytes(b"typedef int o0; this is not C++")
    rc, log = compile_ok(lib, b'#include "my_rope_op.h"\n', 0)
    assert rc != 0 and "error" in log
    rc, log = compile_ok(lib, b'#include "no_such_file.h"\n', 0)
    assert rc != 0 and "no_such_file.h" in log


@pytest.mark.parametrize("spelling", [b'#include <my_op.h>\n', b'#  include   "my_op.h"\n', b'#\tinclude<my_op.h>\n'])
def test_every_spelling_of_a_user_include_bypasses_the_disk_cache(lib, tmp_path, monkeypatch, spelling):
    # the content of a user's file is not in the cache key, whatever the include looks like
    monkeypatch.setenv("SIDEAWARE_CACHE_DIR", str(tmp_path / "cache"))
    (tmp_path / "my_op.h").write_bytes(headers.scale_bias_bf16_header())
    monkeypatch.chdir(tmp_path)
    rc, log = compile_ok(lib, spelling, 0)
    assert rc == 0, log
    (tmp_path / "my_op.h").write_bytes(b"typedef int o0; this is not C++")
    rc, log = compile_ok(lib, spelling, 0)
    assert rc != 0 and "error" in log
    assert not os.path.isdir(tmp_path / "cache") or os.listdir(tmp_path / "cache") == []


def test_headers_of_the_toolchain_are_cached(lib, tmp_path, monkeypatch):
    monkeypatch.setenv("SIDEAWARE_CACHE_DIR", str(tmp_path / "cache"))
    rc, log = compile_ok(lib, b"#include <hip/hip_fp16.h>\n#include <cuda_bf16.h>\n" + headers.fill_header(), 0)
    assert rc == 0, log
    assert len(os.listdir(tmp_path / "cache")) == 1


def test_headers_that_define_the_references_optional_macros_compile(lib):
    # sideaware.cu:60-79: DISCARD_INPUTS with input_discard[4], DYNAMIC_INDEX_FOR_CONCURRENT_KERNELS,
    # FORCE_WRONG_SIDE / FORCE_RANDOM_SIDE: accepted, with no effect on gfx950
    text = lib.sideaware_memcpy_header().decode().replace("#define KERNEL_NAME sideaware_copy", "")
    header = ("#define DISCARD_INPUTS\nconstexpr bool input_discard[4] = {true, false, false, false};\n"
              "#define DYNAMIC_INDEX_FOR_CONCURRENT_KERNELS\n#define FORCE_WRONG_SIDE false\n"
              "#define FORCE_RANDOM_SIDE false\n" + text).encode()
    for variant in (0, 3, 8):
        rc, log = compile_ok(lib, header, variant)
        assert rc == 0, log


def test_aligned_2mib_is_true_only_in_the_aligned_32_bit_instantiations(lib):
    # sideaware.cu:792-794: `aligned_2MiB` goes with the 32-bit index type; a launch whose bases are
    # not 2 MiB-aligned runs an instantiation in which it is false (variant bit 3)
    for variant in range(16):
        block = lib.sideaware_config_block(variant).decode()
        wide, unaligned = variant & 1, variant & 8
        assert ("using size_type = long long;" in block) == bool(wide)
        assert ("constexpr bool aligned_2MiB = true;" in block) == (not wide and not unaligned), variant
        assert ("constexpr bool aligned_2MiB = false;" in block) == bool(wide or unaligned), variant
    header = (b"static_assert(!aligned_2MiB, \"this instantiation is for bases that are not 2 MiB-aligned\");\n"
              + headers.fill_header())
    assert compile_ok(lib, header, 0)[0] != 0
    assert compile_ok(lib, header, 8)[0] == 0
    assert compile_ok(lib, header, 1)[0] == 0


REFERENCE_DIR = "/root/reference"


@pytest.mark.skipif(not os.path.isdir(REFERENCE_DIR), reason="reference checkout not present")
@pytest.mark.parametrize("variant", [0, 1])
def test_reference_rope_header_compiles_unchanged(lib, variant):
    # The reference's own RoPE op header, read as text and handed to this library's compiler.
    with open(os.path.join(REFERENCE_DIR, "kernel_rope.cuh"), "rb") as f:
        rc, log = compile_ok(lib, f.read(), variant)
    assert rc == 0, log


def _isa_of(lib, tmp_path, header, variant):
    """Compiles header + template for gfx950 and returns the disassembly the library wrote."""
    dump = tmp_path / ("isa_%d.txt" % variant)
    if dump.exists():
        dump.unlink()                       # the library appends
    lib.sideaware_write_sass(str(dump).encode())
    try:
        rc, log = compile_ok(lib, header, variant)
        assert rc == 0, log
    finally:
        lib.sideaware_write_sass(b"")
    return dump.read_text()


def _memory_ops(isa, kernel):
    body = isa[isa.index("<%s>:" % kernel):]
    body = body[:body.index("s_endpgm")]
    loads = [l.strip() for l in body.splitlines() if "global_load_dwordx4" in l]
    stores = [l.strip() for l in body.splitlines() if "global_store_dwordx4" in l]
    return loads, stores


def test_cache_policy_is_visible_in_the_isa(lib, tmp_path):
    # the built-in copy: 16-byte loads and stores; the source is marked evict
    assert b"#define SA_IN_PLACE 0" in lib.sideaware_config_block(0)
    assert b"#define SA_IN_PLACE 1" in lib.sideaware_config_block(4)
    loads, stores = _memory_ops(_isa_of(lib, tmp_path, None, 0), "sideaware_copy")
    assert loads and stores
    assert all(" nt" in l for l in loads), loads            # read once: nontemporal
    assert not any(" nt" in s for s in stores), stores        # fits the Infinity Cache: kept for the consumer
    assert all(" sc1" in s for s in stores), stores           # written through the private L2 (agent scope)
    # in place (variant bit 2) with an evict-marked input: the stores stream as well
    loads, stores = _memory_ops(_isa_of(lib, tmp_path, None, 4), "sideaware_copy")
    assert all(" nt" in l for l in loads) and all(" nt" in s for s in stores)
    loads, stores = _memory_ops(_isa_of(lib, tmp_path, None, 2), "sideaware_copy")
    assert all(" nt" in l for l in loads) and all(" nt" in s and " sc1" in s for s in stores)   # larger: everything streams
    # RoPE: the activations stream, the gathered table never does
    rope = headers.rope_header(4096, 32, 0, 128, "bf16", "heads", unrolled=1)
    loads, stores = _memory_ops(_isa_of(lib, tmp_path, rope, 2),
                                "sideaware_rope_fwd_bf16_heads_t4096_h32_0_d128")
    assert sum(" nt" in l for l in loads) == 2 and sum(" nt" not in l for l in loads) == 4, loads
    assert all(" nt" in s for s in stores)
    # a header that fixes the store policy itself gets exactly that, in place or not
    fixed = headers.rope_header(4096, 32, 0, 128, "bf16", "heads", unrolled=1, stream_output=False)
    loads, stores = _memory_ops(_isa_of(lib, tmp_path, fixed, 4),
                                "sideaware_rope_fwd_bf16_heads_t4096_h32_0_d128")
    assert stores and not any(" nt" in s for s in stores) and all(" sc1" in s for s in stores)
    # an expert header names the bits of its 16-byte stores itself
    expert = b'#define SA_STORE_POLICY "sc0 sc1 nt"\n' + headers.memcpy_header()
    loads, stores = _memory_ops(_isa_of(lib, tmp_path, expert, 0), "sideaware_copy_spelled_out")
    assert stores and all(" sc0" in s and " sc1" in s and " nt" in s for s in stores), stores
    # an output that does not start on a 64-byte boundary (variant bit 4): the compiler's stores,
    # which the L2 may merge; streaming ones where the aligned launch would stream
    loads, stores = _memory_ops(_isa_of(lib, tmp_path, None, 16), "sideaware_copy")
    assert stores and not any(" sc1" in s or " nt" in s for s in stores), stores
    loads, stores = _memory_ops(_isa_of(lib, tmp_path, None, 16 | 2), "sideaware_copy")
    assert stores and all(" nt" in s and " sc1" not in s for s in stores), stores
    loads, stores = _memory_ops(_isa_of(lib, tmp_path, expert, 16), "sideaware_copy_spelled_out")
    assert stores and all(" sc0" in s and " sc1" in s and " nt" in s for s in stores), stores   # an expert's bits stand
    # the knob that takes the write-through away: the compiler's stores in every instantiation
    assert lib.sideaware_tune(b"write_through", 0) == 0
    try:
        assert b"#define SA_SPLIT_LINES 1" in lib.sideaware_config_block(0)
        loads, stores = _memory_ops(_isa_of(lib, tmp_path, None, 0), "sideaware_copy")
        assert stores and not any(" sc1" in s or " nt" in s for s in stores), stores
    finally:
        assert lib.sideaware_tune(b"write_through", 1) == 0
    assert b"#define SA_SPLIT_LINES 0" in lib.sideaware_config_block(0)
    # narrower outputs get the same policy on their narrower stores
    mixed = headers.mxfp8_quantize_header()            # bf16 in (16 B per lane), fp8 out (8 B per lane)
    body = _isa_of(lib, tmp_path, mixed, 0)
    narrow = [l for l in body.splitlines() if "global_store_dwordx2" in l]
    assert narrow and all(" sc1" in l for l in narrow), narrow
    # bf16 is narrowed by the hardware's round-to-nearest-even convert, fp32 math is not fused
    isa = _isa_of(lib, tmp_path, rope, 0)
    assert "v_cvt_pk_bf16_f32" in isa and "v_fma_f32" not in isa and "v_pk_mul_f32" not in isa


def test_a_plain_c_program_links_and_runs_against_the_header(lib, tmp_path):
    # the boundary is a C ABI: a C compiler (not C++) must accept include/sideaware.h and the
    # program must link against the shared library
    exe = tmp_path / "c_host"
    lib_dir = os.path.dirname(sa_build.LIB_PATH)
    subprocess.run(["gcc", "-std=c11", "-Wall", "-Werror", os.path.join(ROOT, "tests", "native", "c_host.c"),
                    "-L" + lib_dir, "-l:sideaware.so", "-Wl,-rpath," + lib_dir, "-o", str(exe)], check=True)
    proc = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "c host ok" in proc.stdout


def test_damaged_cache_files_read_as_misses(lib, tmp_path, monkeypatch):
    # the on-disk cache of code objects: a second compile is served from it; a file that was cut
    # short or overwritten is ignored and replaced, never handed to the module loader
    import time
    monkeypatch.setenv("SIDEAWARE_CACHE_DIR", str(tmp_path / "cache"))
    header = headers.fill_header().replace(b"sideaware_fill_int32", b"sideaware_fill_cache_test")
    t0 = time.perf_counter()
    assert compile_ok(lib, header, 0)[0] == 0
    cold = time.perf_counter() - t0
    files = list((tmp_path / "cache").glob("*.co"))
    assert len(files) == 1 and files[0].stat().st_size > 1000
    good = files[0].read_bytes()
    assert good[:4] == b"\x7fELF"
    t0 = time.perf_counter()
    assert compile_ok(lib, header, 0)[0] == 0
    warm = time.perf_counter() - t0
    assert warm < cold / 3, (cold, warm)                       # no compiler run the second time
    for damaged in (good[:len(good) // 2], b"garbage" * 300, good[:-1] + bytes([good[-1] ^ 1]), b""):
        files[0].write_bytes(damaged)
        assert compile_ok(lib, header, 0)[0] == 0
        assert files[0].read_bytes() == good                    # rebuilt: same source, same code object


def test_every_wide_store_is_followed_by_two_wait_states(lib, tmp_path):
    # The 16-byte stores are written as instructions, which the compiler's hazard pass does not
    # look into: the hardware reads a wide store's data registers for two more issue cycles, so
    # each such store must be followed by `s_nop 1` before the compiler's next instruction (which
    # may overwrite them).  Checked over the size / alignment classes and both entry points.
    hn = headers.rope_header(4096, 0, 0, 128, "bf16", "heads", heads_at_launch=True)
    fixed = headers.rope_header(4096, 32, 0, 128, "bf16", "heads")
    seen = 0
    quant = headers.mxfp8_quantize_header()          # its op writes a 16-byte store of its own (the scale bytes)
    for header, variant in ((None, 0), (None, 2), (None, 3), (None, 12), (hn, 4), (hn, 2), (fixed, 4), (fixed, 10),
                            (None, 32), (hn, 32 + 2), (quant, 0), (quant, 2)):
        lines = [l.strip() for l in _isa_of(lib, tmp_path, header, variant).splitlines()]
        lines = [l.split("//")[0].strip() for l in lines if l and not l.startswith(("//", ";"))]
        for i, l in enumerate(lines):
            if l.startswith("global_store_dwordx4") or l.startswith("global_store_dwordx3"):
                seen += 1
                assert lines[i + 1].startswith("s_nop 1"), (variant, lines[i:i + 3])
    assert seen >= 16


def test_half_split_rope_headers_compile_and_refuse_heads_that_would_straddle_a_wave(lib):
    for kw in (dict(dtype="bf16"), dict(dtype="fp32", backward=True), dict(dtype="fp16", heads_first=True),
               dict(dtype="bf16", heads_at_launch=True)):
        for variant in (0, 2, 4):
            rc, log = compile_ok(lib, headers.rope_half_header(4096, 32, 128, **kw), variant)
            assert rc == 0, (kw, variant, log)
    rc, log = compile_ok(lib, headers.rope_half_header(64, 2, 8, "fp32"), 0)      # one vector per half
    assert rc == 0, log
    for bad in ((96, "bf16"), (24, "fp32"), (1024, "fp32"), (7, "fp32")):           # 6 lanes, 3 lanes, 128 lanes, odd
        with pytest.raises(ValueError):
            headers.rope_half_header(16, 2, bad[0], bad[1])


def test_rope_headers_with_per_token_positions_compile(lib):
    for header in (headers.rope_header(1, 32, 0, 128, "bf16", "heads", positions=True),
                   headers.rope_header(1, 0, 0, 64, "fp32", "heads", backward=True, heads_at_launch=True, positions=True),
                   headers.rope_half_header(1, 8, 128, "bf16", positions=True),
                   headers.rope_half_header(1, 0, 128, "fp16", heads_at_launch=True, positions=True)):
        assert b"mem[row" in header
        for variant in (0, 3, 4):
            rc, log = compile_ok(lib, header, variant)
            assert rc == 0, log
    with pytest.raises(ValueError):
        headers.rope_header(16, 4, 2, 64, "fp32", "qkv", positions=True)          # packed QKV has no positions form
    with pytest.raises(ValueError):
        headers.rope_half_header(16, 4, 64, "bf16", heads_first=True, positions=True)
