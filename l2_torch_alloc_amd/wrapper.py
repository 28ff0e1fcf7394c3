"""Python host layer over ``sideaware.so``: ctypes bindings, the PyTorch pluggable allocator and
the ``torch.ops.sideaware.*`` custom ops.

The public names, argument meanings and error behaviour follow the reference's integration
module (``example_wrapper.py:21-187``; the same code is inlined in ``test.py:14-157``):
``sideaware_init``, ``sideaware_enabled``, ``sideaware_create_kernel``, ``sideaware_info``,
``sideaware_info_raw``, ``sideaware_torch_side_index``, ``sideaware_gpu_side_index``,
``sideaware_cpu_side_index`` and the three ops ``memcpy`` / ``one_to_one`` / ``elementwise``.
A script written against the reference module runs against this one.

There is no CPU fallback anywhere in this file: without the built library, or without a GPU,
the calls raise.
"""
from __future__ import annotations

import ctypes
import os
import sys
from typing import Optional

import torch

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
DEFAULT_LIBRARY = os.path.join(_PKG_DIR, "sideaware.so")

_lib: Optional[ctypes.CDLL] = None
_ops_registered = False
_allocator_installed = False
_info = (0, 0, 0, 0, 0)
_info_str = {"num_sms": 0, "side0": 0, "side1": 0, "min": 0, "hash": 0}
_torch_side_index = None
_gpu_side_index = None
_cpu_side_index = None

_vp, _ci, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t

# name -> (restype, argtypes).  Widths are those of include/sideaware.h.  Note the reference's
# Python binding declares sideband_value as a pointer-sized integer (test.py:36); both widths
# travel in the same integer register on x86-64, so either declaration works.
_SIGNATURES = {
    "sideaware_malloc_auto": (_vp, [_sz, _ci, _vp]),
    "sideaware_malloc_auto_raising": (_vp, [_sz, _ci, _vp]),
    "sideaware_free_auto": (None, [_vp, _sz, _ci, _vp]),
    "sideaware_malloc": (_ci, [ctypes.POINTER(_vp), _sz]),
    "sideaware_free": (_ci, [_vp]),
    "sideaware_malloc_async": (_ci, [ctypes.POINTER(_vp), _sz, _vp]),
    "sideaware_free_async": (_ci, [_vp, _vp]),
    "sideaware_release_unused": (_sz, []),
    "sideaware_create_kernel": (_ci, [ctypes.c_char_p]),
    "sideaware_create_kernel_advanced": (_ci, [ctypes.c_char_p, ctypes.c_bool, _ci]),
    "sideaware_elementwise": (None, [_ci, _sz, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _vp]),
    "sideaware_one_to_one": (None, [_ci, _sz, _vp, _vp, _ci, _vp]),
    "sideaware_memcpy": (None, [_vp, _vp, _sz, _ci, _vp]),
    "sideaware_compression": (None, [ctypes.c_bool]),
    "sideaware_alloc_threshold": (None, [_sz]),
    "sideaware_prealloc_config": (None, [_ci, _ci]),
    "sideaware_free_mapped_thresholds": (None, [_sz, _sz]),
    "sideaware_write_sass": (None, [ctypes.c_char_p]),
    "sideaware_fill_side_index": (None, [_vp]),
    "sideaware_gpu_side_index": (_vp, []),
    "sideaware_cpu_side_index": (_vp, []),
    "sideaware_sm_side_summary": (ctypes.POINTER(ctypes.c_int * 5), []),
    "sideaware_num_sms": (_ci, []),
    "sideaware_num_sm_side0": (_ci, []),
    "sideaware_num_sm_side1": (_ci, []),
    "sideaware_min_sm_per_side": (_ci, []),
    "sideaware_hash_mask": (_ci, []),
    "sideaware_elementwise_batch": (None, [_ci, _ci, _vp, _ci, _vp]),
    "sideaware_reserve_limit": (None, [_sz]),
    "sideaware_oom_raises": (None, [_ci]),
    "sideaware_arena_bytes": (None, [_sz]),
    "sideaware_num_xcds": (_ci, []),
    "sideaware_xcd_dealing_verified": (_ci, []),
    "sideaware_probe_sides": (_ci, [_vp, _sz, ctypes.c_ulonglong, _ci, _vp, _ci, _vp]),
    "sideaware_probe_sides_noalloc": (_ci, [_vp, _sz, ctypes.c_ulonglong, _ci, _vp, _ci, _vp]),
    "sideaware_register_region": (_ci, [_vp, _sz, _ci]),
    "sideaware_unregister_region": (None, [_vp, _ci]),
    "sideaware_side_address_mask": (ctypes.c_ulonglong, []),
    "sideaware_side_of": (_ci, [_vp]),
    "sideaware_stream_dealing": (_ci, [_vp]),
    "sideaware_set_stream_dealing": (None, [_vp, _ci]),
    "sideaware_launch_counts": (None, [ctypes.POINTER(ctypes.c_ulonglong), ctypes.POINTER(ctypes.c_ulonglong)]),
    "sideaware_last_error": (ctypes.c_char_p, []),
    "sideaware_clear_error": (None, []),
    "sideaware_compile_check": (_ci, [ctypes.c_char_p, _ci, ctypes.c_char_p, _sz]),
    "sideaware_kernel_source": (ctypes.c_char_p, []),
    "sideaware_memcpy_header": (ctypes.c_char_p, []),
    "sideaware_config_block": (ctypes.c_char_p, [_ci]),
    "sideaware_kernel_info": (_ci, [_ci, _ci, ctypes.POINTER(_ci)]),
    "sideaware_alloc_stats": (_ci, [ctypes.POINTER(ctypes.c_ulonglong), _ci]),
    "sideaware_tune": (_ci, [ctypes.c_char_p, ctypes.c_longlong]),
    "sideaware_tune_get": (ctypes.c_longlong, [ctypes.c_char_p]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

POOL_STAT_FIELDS = (
    "large_hits", "large_misses", "small_hits", "small_carves", "slabs_acquired", "backing_acquires",
    "backing_releases", "stream_syncs", "device_syncs", "trims", "ladder_retries", "failures",
    "foreign_frees", "bytes_live", "bytes_cached_large", "bytes_cached_small", "bytes_reserved",
    "peak_reserved", "large_carves", "arenas_acquired", "bytes_free_arena", "bytes_free_slab_arena",
    "cache_folds", "refused_frees", "canonical_placements",
)


def bind(path: str = DEFAULT_LIBRARY) -> ctypes.CDLL:
    """dlopen the library and declare every entry point's C signature.  Touches no device."""
    if not os.path.exists(path):
        raise FileNotFoundError(
            "%s is not built; run `python -m l2_torch_alloc_amd.build` (needs hipcc)" % path)
    lib = ctypes.CDLL(path)
    for name, (restype, argtypes) in _SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if the library lacks a declared symbol
        fn.restype = restype
        fn.argtypes = argtypes
    return lib


def library() -> ctypes.CDLL:
    if _lib is None:
        raise RuntimeError("sideaware is not initialised: call sideaware_init() first")
    return _lib


# ------------------------------------------------------------------------------------------------
# Externally visible API (plus torch.ops.sideaware.[memcpy/one_to_one/elementwise])
# ------------------------------------------------------------------------------------------------

def sideaware_enabled() -> int:
    return 1 if _lib is not None else 0


def sideaware_create_kernel(header_code: bytes) -> int:
    """Registers an op header; returns the id to pass to one_to_one / elementwise."""
    return library().sideaware_create_kernel(header_code)


def sideaware_torch_side_index():
    """torch.uint8 tensor with one entry per CU; before ``sideaware_init`` a one-element zero
    tensor, as in the reference (``example_wrapper.py:29-33``)."""
    global _torch_side_index
    if _torch_side_index is None:
        _torch_side_index = torch.zeros(1, dtype=torch.uint8, device="cuda")
    return _torch_side_index


def sideaware_gpu_side_index():
    return _gpu_side_index          # device address of the library's own copy


def sideaware_cpu_side_index():
    return _cpu_side_index          # host address of the library's own copy


def sideaware_info():
    return _info_str                # {"num_sms", "side0", "side1", "min", "hash"}


def sideaware_info_raw():
    return _info                    # (num_sms, side0, side1, min, hash)


def sideaware_last_error() -> str:
    return library().sideaware_last_error().decode()


def sideaware_alloc_stats() -> dict:
    buf = (ctypes.c_ulonglong * len(POOL_STAT_FIELDS))()
    n = library().sideaware_alloc_stats(buf, len(POOL_STAT_FIELDS))
    return {POOL_STAT_FIELDS[i]: int(buf[i]) for i in range(n)}


def sideaware_init(path: str = DEFAULT_LIBRARY, install_allocator: bool = True) -> None:
    """Loads the library, routes PyTorch's device allocations through it and registers the ops.

    Must run before the process's first device allocation when ``install_allocator`` is true
    (PyTorch refuses to swap allocators later), exactly like the reference's ``sideaware_init``.
    Safe to call again: later calls only refresh the metadata.
    """
    global _lib, _allocator_installed
    if not torch.cuda.is_available():
        raise RuntimeError("sideaware needs a GPU: torch.cuda.is_available() is False")
    path = os.path.abspath(path)
    if install_allocator and not _allocator_installed:
        # PyTorch does not check the pointer its pluggable allocator returns: it gets the entry point
        # that raises (a RuntimeError in Python) when the pool is exhausted instead of returning null.
        # sideaware_malloc_auto itself keeps the reference's contract (null), for ctypes callers.
        allocator = torch.cuda.memory.CUDAPluggableAllocator(path, "sideaware_malloc_auto_raising", "sideaware_free_auto")
        torch.cuda.memory.change_current_allocator(allocator)
        _allocator_installed = True
    if _lib is None:
        _lib = bind(path)
    _register_ops()
    _refresh_metadata()
    # the reference prints this line when initialisation is done (example_wrapper.py:109); here it
    # goes to stderr so that programs with a machine-readable stdout can use the module
    print("L2 Side Aware metadata: %s" % (_info_str,), file=sys.stderr)


def _refresh_metadata() -> None:
    global _info, _info_str, _torch_side_index, _gpu_side_index, _cpu_side_index
    lib = library()
    _info = tuple(lib.sideaware_sm_side_summary().contents)
    if _info[0] <= 0:
        raise RuntimeError("sideaware failed to initialise the device: " + sideaware_last_error())
    _info_str = {"num_sms": _info[0], "side0": _info[1], "side1": _info[2], "min": _info[3], "hash": _info[4]}
    _torch_side_index = torch.zeros(_info[0], dtype=torch.uint8, device="cuda")
    lib.sideaware_fill_side_index(_torch_side_index.data_ptr())
    _gpu_side_index = lib.sideaware_gpu_side_index()
    _cpu_side_index = lib.sideaware_cpu_side_index()


# ------------------------------------------------------------------------------------------------
# The three ops.  Exposed through torch.ops.sideaware.* so that they trace under torch.compile.
# ------------------------------------------------------------------------------------------------

# The raw handle of the current stream of a device without building a torch.cuda.Stream object
# (a third of the cost of a small launch); older PyTorch builds lack the private accessor.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _device_and_stream(t: Optional[torch.Tensor] = None):
    """(device index, current stream handle): of the device the given tensor lives on, or of the
    current device."""
    device = t.get_device() if t is not None else torch.cuda.current_device()
    if _raw_stream is not None:
        return device, _raw_stream(device)
    return device, torch.cuda.current_stream(device).cuda_stream


def _check(t: Optional[torch.Tensor], name: str) -> int:
    """Address of a contiguous, 16-byte aligned device tensor; 0 for None."""
    if t is None:
        return 0
    assert t.is_cuda, name + " must be on the GPU"
    assert t.is_contiguous(), name + " must be contiguous"
    ptr = t.data_ptr()
    assert not ptr & 15, name + " must be 16-byte aligned"
    return ptr


def sideaware_memcpy(dst: torch.Tensor, src: torch.Tensor) -> None:
    assert dst.dtype == src.dtype, "Source and destination must have the same dtype"
    assert dst.numel() >= src.numel(), "Destination tensor must be at least as large as source"
    dst_ptr, src_ptr = _check(dst, "dst"), _check(src, "src")
    device, stream = _device_and_stream(dst)
    (_lib or library()).sideaware_memcpy(dst_ptr, src_ptr, src.numel() * src.element_size(), device, stream)


def sideaware_one_to_one(kernel_id: int, dst: torch.Tensor, src: Optional[torch.Tensor]) -> None:
    # The byte count is taken from dst, as the reference does (test.py:92-94).
    num_bytes = dst.numel() * dst.element_size() if dst is not None else 0
    assert num_bytes > 0
    dst_ptr, src_ptr = _check(dst, "dst"), _check(src, "src")
    device, stream = _device_and_stream(dst)
    (_lib or library()).sideaware_one_to_one(kernel_id, num_bytes, dst_ptr, src_ptr, device, stream)


def sideaware_elementwise(kernel_id: int,
                          out0: Optional[torch.Tensor], out1: Optional[torch.Tensor],
                          out2: Optional[torch.Tensor], out3: Optional[torch.Tensor],
                          in0: Optional[torch.Tensor], in1: Optional[torch.Tensor],
                          in2: Optional[torch.Tensor], in3: Optional[torch.Tensor],
                          sideband_tensor: Optional[torch.Tensor] = None, sideband_value: int = 0,
                          parallel_chunks: int = 0, forced_sm_per_side: int = 0) -> None:
    # The byte count is taken from out0, as the reference does (test.py:114-116).
    num_bytes = out0.numel() * out0.element_size() if out0 is not None else 0
    assert num_bytes > 0
    o0, o1, o2, o3 = _check(out0, "out0"), _check(out1, "out1"), _check(out2, "out2"), _check(out3, "out3")
    i0, i1, i2, i3 = _check(in0, "in0"), _check(in1, "in1"), _check(in2, "in2"), _check(in3, "in3")
    device, stream = _device_and_stream(out0)            # after the checks: out0 is on a GPU
    (_lib or library()).sideaware_elementwise(
        kernel_id, num_bytes, o0, o1, o2, o3, i0, i1, i2, i3,
        sideband_tensor.data_ptr() if sideband_tensor is not None else 0, sideband_value,
        parallel_chunks, forced_sm_per_side, device, stream)


_op_library = None


def _register_ops() -> None:
    global _ops_registered, _op_library
    if _ops_registered:
        return
    _op_library = torch.library.Library("sideaware", "FRAGMENT")
    for name, fn, mutated in (
        ("memcpy", sideaware_memcpy, ["dst"]),
        ("one_to_one", sideaware_one_to_one, ["dst"]),
        ("elementwise", sideaware_elementwise, ["out0", "out1", "out2", "out3", "sideband_tensor"]),
    ):
        schema = torch.library.infer_schema(fn, mutates_args=mutated)
        _op_library.define(name + schema)
        _op_library.impl(name, fn, "CUDA")
    _ops_registered = True
