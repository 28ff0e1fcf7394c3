"""A host program that binds the library the way the reference's own script does, run by
tests/test_gpu_reference_binding.py in a fresh process whose working directory holds `./sideaware.so`.

What is taken from the reference's script (test.py:14-39, 86, 104, 141) is the calling convention, not
its text: the library is opened by a path relative to the working directory, both through
PyTorch's pluggable allocator and through ctypes; `sideband_value` is declared pointer-sized; the
stream argument is the `torch.cuda.Stream` object itself (ctypes takes its `_as_parameter_`); the three
ops are registered in the `sideaware` torch library so that they trace under torch.compile.  Every
check prints one `ok:` line; any failure ends the process with a non-zero status.
"""
import ctypes
import sys
from typing import Optional

import torch

LIB_PATH = "./sideaware.so"

torch.cuda.memory.change_current_allocator(
    torch.cuda.memory.CUDAPluggableAllocator(LIB_PATH, "sideaware_malloc_auto", "sideaware_free_auto"))
lib = ctypes.CDLL(LIB_PATH)

P, I, Z = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
for name, restype, argtypes in (
        ("sideaware_create_kernel", I, [ctypes.c_char_p]),
        ("sideaware_sm_side_summary", ctypes.POINTER(I * 5), []),
        ("sideaware_fill_side_index", None, [P]),
        ("sideaware_memcpy", None, [P, P, Z, I, P]),
        ("sideaware_one_to_one", None, [I, Z, P, P, I, P]),
        # kernel, bytes, four outputs, four inputs, sideband pointer, sideband value (pointer-sized
        # in the reference's binding), groups, forced per side, device, stream
        ("sideaware_elementwise", None, [I, Z, P, P, P, P, P, P, P, P, P, P, I, I, I, P])):
    fn = getattr(lib, name)
    fn.restype, fn.argtypes = restype, argtypes


def here():
    return torch.cuda.current_device(), torch.cuda.current_stream()      # the Stream object, not its handle


def ptr(t):
    return 0 if t is None else t.data_ptr()


def op_memcpy(dst: torch.Tensor, src: torch.Tensor) -> None:
    assert dst.is_contiguous() and src.is_contiguous()
    nbytes = dst.numel() * dst.element_size()
    assert nbytes == src.numel() * src.element_size() and ptr(dst) % 16 == 0 and ptr(src) % 16 == 0
    device, stream = here()
    lib.sideaware_memcpy(ptr(dst), ptr(src), nbytes, device, stream)


def op_one_to_one(kernel_id: int, dst: torch.Tensor, src: torch.Tensor) -> None:
    device, stream = here()
    lib.sideaware_one_to_one(kernel_id, dst.numel() * dst.element_size(), ptr(dst), ptr(src), device, stream)


def op_elementwise(kernel_id: int,
                   out0: torch.Tensor, out1: Optional[torch.Tensor], out2: Optional[torch.Tensor],
                   out3: Optional[torch.Tensor],
                   in0: Optional[torch.Tensor], in1: Optional[torch.Tensor], in2: Optional[torch.Tensor],
                   in3: Optional[torch.Tensor],
                   sideband_tensor: Optional[torch.Tensor] = None, sideband_value: int = 0,
                   parallel_chunks: int = 0, forced_sm_per_side: int = 0) -> None:
    device, stream = here()
    lib.sideaware_elementwise(kernel_id, out0.numel() * out0.element_size(),
                              ptr(out0), ptr(out1), ptr(out2), ptr(out3), ptr(in0), ptr(in1), ptr(in2), ptr(in3),
                              ptr(sideband_tensor), sideband_value, parallel_chunks, forced_sm_per_side, device, stream)


ops = torch.library.Library("sideaware", "FRAGMENT")
for op_name, fn, mutated in (("memcpy", op_memcpy, ["dst"]), ("one_to_one", op_one_to_one, ["dst"]),
                             ("elementwise", op_elementwise, ["out0", "out1", "out2", "out3", "sideband_tensor"])):
    ops.define(op_name + torch.library.infer_schema(fn, mutates_args=mutated))
    ops.impl(op_name, fn, "CUDA")


def check(what, ok):
    print(("ok: " if ok else "FAILED: ") + what, flush=True)
    if not ok:
        sys.exit(1)


# metadata (test.py:163-164)
summary = tuple(lib.sideaware_sm_side_summary().contents)
check("summary names %d compute units, %d + %d per side, hash 0x%x" % (summary[0], summary[1], summary[2], summary[4]),
      summary[0] > 0 and summary[1] > 0 and summary[3] > 0)
index = torch.zeros(summary[0], dtype=torch.uint8, device="cuda")
lib.sideaware_fill_side_index(index.data_ptr())
torch.cuda.synchronize()
check("side index tensor filled", int(index.max()) > 0)

# an 8 x 8 fp32 copy, eager and inside a compiled function with no graph break (test.py:166-184)
src = torch.ones((8, 8), dtype=torch.float32, device="cuda")
dst = torch.zeros_like(src)
torch.ops.sideaware.memcpy(dst, src)
check("eager 8x8 copy", bool(torch.all(dst == 1.0)))


@torch.compile(fullgraph=True)
def compiled_copy(d, s):
    torch.ops.sideaware.memcpy(d, s)
    return d


src2 = torch.ones((8, 8), dtype=torch.float32, device="cuda") * 2.0
dst2 = torch.zeros_like(src2)
out = compiled_copy(dst2, src2)
check("8x8 copy under torch.compile(fullgraph=True)", bool(torch.all(dst2 == 2.0)) and out.data_ptr() == dst2.data_ptr())

# a header written for the reference: CUDA type names, two inputs and two outputs of four
# different types, reversed traversal, every input marked evict (test.py:191-230)
header = b"""
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
                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3)
{
    out0 = (o0)((float)in0 + (float)in1);
    out1 = (o1)((float)in1 * 10.0f);
}
constexpr bool reverse_order = true;
constexpr bool input_evict[4] = {1,1,1,1};
"""
a = torch.arange(64, device="cuda", dtype=torch.float32).reshape(8, 8).to(torch.bfloat16)
b = torch.full((8, 8), 2.0, device="cuda")
sum_out = torch.zeros((8, 8), device="cuda")
ten_out = torch.zeros((8, 8), device="cuda", dtype=torch.float16)
kernel_id = lib.sideaware_create_kernel(header)
torch.ops.sideaware.elementwise(kernel_id, sum_out, ten_out, None, None, a, b, None, None, None, 0, 0, 0)
check("run-time compiled mixed-type op (kernel id %d)" % kernel_id,
      kernel_id > 0 and bool(torch.all(sum_out == (a + b))) and bool(torch.all(ten_out == (b * 10.0))))


def copy_matches_torch(shape, dtype, start=0):
    n = 1
    for d in shape:
        n *= d
    s = torch.arange(n, dtype=dtype, device="cuda").reshape(shape)
    mine, theirs = torch.zeros_like(s), torch.zeros_like(s)
    torch.ops.sideaware.memcpy(mine[start:], s[start:])
    theirs[start:].copy_(s[start:])
    return bool(torch.all(mine == theirs))


# the shapes of the reference's copy tests that fit a short run (test.py:310-318)
check("(4, 777) fp32: 12,432 bytes, a tail only", copy_matches_torch((4, 777), torch.float32))
check("(1000, 1000) int16", copy_matches_torch((1000, 1000), torch.int16))
check("(1000, 1000) float64", copy_matches_torch((1000, 1000), torch.float64))
check("(10000, 1000) fp32, 40 MB", copy_matches_torch((10000, 1000), torch.float32))
check("(20000, 20000) fp32, 1.6 GB", copy_matches_torch((20000, 20000), torch.float32))
print("done", flush=True)
