"""ctypes/numpy front end of the CPU oracle (``rope_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``; the shipped library and its Python host layer never
import it.

Every function here is a thin array wrapper around the C restatement of the reference's CPU
code (``example_llmc_rope.cu:19-86``, ``:166-195``; ``kernel_rope.cuh:29-60``).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile ``liboracle.so`` with gcc (a second or so)."""
    if force or not os.path.exists(_LIB_PATH) or (
        os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "rope_oracle.c"))
    ):
        subprocess.run(["make", "-C", _HERE, "-B", "liboracle.so"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, ci, cf, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t
        L.oracle_f32_to_bf16_array.argtypes = [vp, vp, sz]
        L.oracle_bf16_to_f32_array.argtypes = [vp, vp, sz]
        L.oracle_freqs_cis.argtypes = [vp, ci, ci, cf, ci]
        L.oracle_rope_forward_qkv_f32.argtypes = [vp, vp, vp, ci, ci, ci, ci, ci]
        L.oracle_rope_backward_qkv_f32.argtypes = [vp, vp, vp, ci, ci, ci, ci, ci]
        L.oracle_rope_forward_heads_f32.argtypes = [vp, vp, vp, ci, ci, ci, ci]
        L.oracle_rope_backward_heads_f32.argtypes = [vp, vp, vp, ci, ci, ci, ci]
        L.oracle_rope_forward_heads_bf16.argtypes = [vp, vp, vp, ci, ci, ci, ci]
        L.oracle_scale_bias_bf16.argtypes = [vp, vp, cf, cf, sz]
        L.oracle_memcpy.argtypes = [vp, vp, sz]
        L.oracle_mxfp8_quantize.argtypes = [vp, vp, vp, sz]
        L.oracle_mxfp8_dequantize.argtypes = [vp, vp, vp, sz]
        L.oracle_f32_to_e4m3.argtypes = [cf]
        L.oracle_f32_to_e4m3.restype = ctypes.c_uint8
        L.oracle_e4m3_to_f32.argtypes = [ctypes.c_uint8]
        L.oracle_e4m3_to_f32.restype = cf
        L.oracle_validate_f32.argtypes = [vp, vp, sz, cf]
        L.oracle_validate_f32.restype = sz
        for name in ("oracle_f32_to_bf16_array", "oracle_bf16_to_f32_array", "oracle_freqs_cis",
                     "oracle_rope_forward_qkv_f32", "oracle_rope_backward_qkv_f32",
                     "oracle_rope_forward_heads_f32", "oracle_rope_backward_heads_f32",
                     "oracle_rope_forward_heads_bf16", "oracle_scale_bias_bf16", "oracle_memcpy",
                     "oracle_mxfp8_quantize", "oracle_mxfp8_dequantize"):
            getattr(L, name).restype = None
        _lib = L
    return _lib


def _p(a: np.ndarray) -> int:
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _u16(a) -> np.ndarray:
    a = np.ascontiguousarray(a)
    assert a.dtype == np.uint16, "bf16 data travels as its uint16 bit pattern"
    return a


def f32_to_bf16(x) -> np.ndarray:
    """fp32 array -> bf16 bit patterns (uint16), round to nearest even."""
    x = _f32(x)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().oracle_f32_to_bf16_array(_p(out), _p(x), x.size)
    return out


def bf16_to_f32(h) -> np.ndarray:
    h = _u16(h)
    out = np.empty(h.shape, dtype=np.float32)
    lib().oracle_bf16_to_f32_array(_p(out), _p(h), h.size)
    return out


def freqs_cis(head_dim: int, end: int, theta: float, use_scaled: bool = False) -> np.ndarray:
    """(end, head_dim) fp32 table, cos at even and sin at odd columns."""
    out = np.empty((end, head_dim), dtype=np.float32)
    lib().oracle_freqs_cis(_p(out), head_dim, end, float(theta), int(use_scaled))
    return out


def rope_forward_qkv_f32(inp, freqs, Nq: int, Nkv: int) -> np.ndarray:
    """inp (B, T, Nq+2*Nkv, HS) fp32 -> rotated q,k heads, copied v heads."""
    inp, freqs = _f32(inp), _f32(freqs)
    B, T, N, HS = inp.shape
    assert N == Nq + 2 * Nkv and freqs.shape == (T, HS)
    out = np.empty_like(inp)
    lib().oracle_rope_forward_qkv_f32(_p(out), _p(inp), _p(freqs), B, T, Nq, Nkv, HS)
    return out


def rope_backward_qkv_f32(dout, freqs, Nq: int, Nkv: int) -> np.ndarray:
    dout, freqs = _f32(dout), _f32(freqs)
    B, T, N, HS = dout.shape
    assert N == Nq + 2 * Nkv and freqs.shape == (T, HS)
    dinp = np.zeros_like(dout)
    lib().oracle_rope_backward_qkv_f32(_p(dinp), _p(dout), _p(freqs), B, T, Nq, Nkv, HS)
    return dinp


def rope_forward_heads_f32(inp, freqs) -> np.ndarray:
    """inp (B, T, NH, HS) fp32, every head rotated."""
    inp, freqs = _f32(inp), _f32(freqs)
    B, T, NH, HS = inp.shape
    assert freqs.shape == (T, HS)
    out = np.empty_like(inp)
    lib().oracle_rope_forward_heads_f32(_p(out), _p(inp), _p(freqs), B, T, NH, HS)
    return out


def rope_backward_heads_f32(dout, freqs) -> np.ndarray:
    dout, freqs = _f32(dout), _f32(freqs)
    B, T, NH, HS = dout.shape
    assert freqs.shape == (T, HS)
    dinp = np.empty_like(dout)
    lib().oracle_rope_backward_heads_f32(_p(dinp), _p(dout), _p(freqs), B, T, NH, HS)
    return dinp


def rope_forward_heads_bf16(inp_bits, freqs) -> np.ndarray:
    """inp_bits (B, T, NH, HS) uint16 bf16 bit patterns -> rotated, RNE-rounded bit patterns."""
    inp_bits, freqs = _u16(inp_bits), _f32(freqs)
    B, T, NH, HS = inp_bits.shape
    assert freqs.shape == (T, HS)
    out = np.empty_like(inp_bits)
    lib().oracle_rope_forward_heads_bf16(_p(out), _p(inp_bits), _p(freqs), B, T, NH, HS)
    return out


def scale_bias_bf16(x_bits, scale: float, bias: float) -> np.ndarray:
    x_bits = _u16(x_bits)
    out = np.empty_like(x_bits)
    lib().oracle_scale_bias_bf16(_p(out), _p(x_bits), float(scale), float(bias), x_bits.size)
    return out


def mxfp8_quantize(x_bits):
    """bf16 bit patterns (count a multiple of 32) -> (E4M3 bytes, E8M0 scale bytes, one per 32)."""
    x_bits = _u16(x_bits)
    assert x_bits.size % 32 == 0
    q = np.empty(x_bits.shape, dtype=np.uint8)
    scales = np.empty(x_bits.size // 32, dtype=np.uint8)
    lib().oracle_mxfp8_quantize(_p(q), _p(scales), _p(x_bits), x_bits.size)
    return q, scales


def mxfp8_dequantize(q, scales) -> np.ndarray:
    q = np.ascontiguousarray(q, dtype=np.uint8)
    scales = np.ascontiguousarray(scales, dtype=np.uint8)
    assert q.size == scales.size * 32
    out = np.empty(q.shape, dtype=np.uint16)
    lib().oracle_mxfp8_dequantize(_p(out), _p(q), _p(scales), q.size)
    return out


def f32_to_e4m3(values) -> np.ndarray:
    L = lib()
    return np.array([L.oracle_f32_to_e4m3(float(v)) for v in np.asarray(values, dtype=np.float32).ravel()],
                    dtype=np.uint8)


def e4m3_to_f32(codes) -> np.ndarray:
    L = lib()
    return np.array([L.oracle_e4m3_to_f32(int(c)) for c in np.asarray(codes, dtype=np.uint8).ravel()],
                    dtype=np.float32)


def memcpy(src: np.ndarray) -> np.ndarray:
    src = np.ascontiguousarray(src)
    out = np.empty_like(src)
    lib().oracle_memcpy(_p(out), _p(src), src.nbytes)
    return out


def validate_f32(got, ref, tolerance: float = 1e-5) -> int:
    """Fault count under llm.c's rule: |ref-got| > tol + |ref|*FLT_EPSILON."""
    got, ref = _f32(got), _f32(ref)
    assert got.shape == ref.shape
    return int(lib().oracle_validate_f32(_p(got), _p(ref), ref.size, float(tolerance)))


def bf16_ulp_distance(a_bits, b_bits) -> np.ndarray:
    """Distance in bf16 units-in-the-last-place between two bit-pattern arrays.

    Maps sign-magnitude patterns onto a monotone integer line first, so the distance is
    right across zero and across binades.
    """
    def line(x):
        x = x.astype(np.int32)
        return np.where(x & 0x8000, -(x & 0x7FFF), x & 0x7FFF)
    return np.abs(line(_u16(a_bits)) - line(_u16(b_bits)))


# ----------------------------------------------------------------------------------------------
# Half-split pair layout ("rotate_half": element i of a head pairs with element i + HS/2).  The
# reference has only the interleaved layout (kernel_rope.cuh:29-60, example_llmc_rope.cu:54-86);
# the half-split op is the same rotation applied to a permuted head, so it is stated here as
# exactly that: permute, run the restated reference loop, permute back.  tests/test_oracle.py pins
# it against the formula written out directly (x1*c - x2*s, x2*c + x1*s) in numpy float32, bit for
# bit, and against a float64 complex product.

def _half_to_interleaved(x: np.ndarray) -> np.ndarray:
    h = x.shape[-1] // 2
    return np.ascontiguousarray(np.stack([x[..., :h], x[..., h:]], axis=-1).reshape(x.shape))


def _interleaved_to_half(y: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(np.concatenate([y[..., 0::2], y[..., 1::2]], axis=-1))


def _bthd(x: np.ndarray, heads_first: bool) -> np.ndarray:
    return np.ascontiguousarray(np.swapaxes(x, 1, 2)) if heads_first else x


def rope_half_forward_heads_f32(inp, freqs, heads_first: bool = False) -> np.ndarray:
    """inp (B, T, NH, HS) fp32, or (B, NH, T, HS) with heads_first; freqs as for the interleaved op."""
    y = rope_forward_heads_f32(_half_to_interleaved(_bthd(_f32(inp), heads_first)), freqs)
    return _bthd(_interleaved_to_half(y), heads_first)


def rope_half_backward_heads_f32(dout, freqs, heads_first: bool = False) -> np.ndarray:
    y = rope_backward_heads_f32(_half_to_interleaved(_bthd(_f32(dout), heads_first)), freqs)
    return _bthd(_interleaved_to_half(y), heads_first)


def rope_half_forward_heads_bf16(inp_bits, freqs, heads_first: bool = False) -> np.ndarray:
    y = rope_forward_heads_bf16(_half_to_interleaved(_bthd(_u16(inp_bits), heads_first)), freqs)
    return _bthd(_interleaved_to_half(y), heads_first)
