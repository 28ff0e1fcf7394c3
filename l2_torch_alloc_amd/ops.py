"""Ready-made ops on top of ``torch.ops.sideaware.elementwise``: RoPE (llm.c formula), bf16
scale+bias and fill.  Each builds its op header once per shape (``headers.py``), registers it with
the library and launches through the same custom op a user-written header would use.

The frequency table is an *input*: build it on the host with ``freqs_cis_table`` (the llm.c
formula, ``example_llmc_rope.cu:19-52``) or bring your own, as (T, head_dim) fp32 with cos at
even and sin at odd columns.
"""
from __future__ import annotations

import ctypes
import math
import os
from typing import Dict, Optional, Tuple

import torch

from . import headers, wrapper

_kernel_ids: Dict[Tuple, int] = {}
_CHECK_POSITION_VALUES = os.environ.get("SIDEAWARE_CHECK_POSITIONS") == "1"

_HEADER_BUILDERS = {
    "rope": headers.rope_header,
    "rope_half": headers.rope_half_header,
    "scale_bias_bf16": headers.scale_bias_bf16_header,
    "mxfp8_quantize": headers.mxfp8_quantize_header,
    "mxfp8_dequantize": headers.mxfp8_dequantize_header,
    "fill": headers.fill_header,
}


@torch.compiler.assume_constant_result
def _kernel(builder: str, args: Tuple = (), kwargs: Tuple = ()) -> int:
    """The kernel id of the op whose header is ``_HEADER_BUILDERS[builder](*args, **dict(kwargs))``,
    registering it on first use.  Everything it takes is a constant (strings, ints, bools), so a
    tracer evaluates the call once, while it traces, and keeps the id as a constant of the graph:
    an op whose first use falls inside ``torch.compile(fullgraph=True)`` needs no eager warm-up."""
    key = (builder, args, kwargs)
    kid = _kernel_ids.get(key)
    if kid is None:
        kid = wrapper.sideaware_create_kernel(_HEADER_BUILDERS[builder](*args, **dict(kwargs)))
        _kernel_ids[key] = kid
    return kid


def _elementwise(*args) -> None:
    """The elementwise op.  Eager code goes straight to the op's implementation, the function
    ``torch.ops.sideaware.elementwise`` dispatches to, and saves the dispatcher's per-call cost
    (about a microsecond of a small launch); under ``torch.compile`` the call goes through the
    registered op, which the tracer keeps as one opaque node."""
    if torch.compiler.is_compiling():
        torch.ops.sideaware.elementwise(*args)
    else:
        wrapper.sideaware_elementwise(*args)


def freqs_cis_table(head_dim: int, end: int, theta: float, use_scaled: bool = False) -> torch.Tensor:
    """(end, head_dim) fp32 table on the host: [t, 2i] = cos(t*f_i), [t, 2i+1] = sin(t*f_i),
    f_i = theta^(-2i/head_dim) in fp32, optionally with the Llama-3.1 wavelength rescaling
    (``example_llmc_rope.cu:25-43``).  Built with torch CPU ops in fp32."""
    i = torch.arange(head_dim // 2, dtype=torch.float32)
    freq = 1.0 / torch.pow(torch.tensor(theta, dtype=torch.float32), (2 * i) / head_dim)
    if use_scaled:
        scale_factor, low_factor, high_factor, old_len = 8.0, 1.0, 4.0, 8192.0
        wavelen = (2.0 * math.pi / freq.double()).float()
        smooth = (old_len / wavelen - low_factor) / (high_factor - low_factor)
        blended = (1.0 - smooth) * freq / scale_factor + smooth * freq
        freq = torch.where(wavelen < old_len / high_factor, freq,
                           torch.where(wavelen > old_len / low_factor, freq / scale_factor, blended))
    angle = torch.arange(end, dtype=torch.float32)[:, None] * freq[None, :]
    table = torch.empty(end, head_dim, dtype=torch.float32)
    table[:, 0::2] = torch.cos(angle)
    table[:, 1::2] = torch.sin(angle)
    return table


_ROPE_DTYPES = {torch.float32: "fp32", torch.bfloat16: "bf16", torch.float16: "fp16"}


def _check_positions(positions: torch.Tensor, tokens: int, x: torch.Tensor, rows: int) -> None:
    """The kernel reads table row ``positions[token]`` without a bound (a check per element would
    cost more than the op): shape, type and device are checked here, and with
    ``SIDEAWARE_CHECK_POSITIONS=1`` in the environment the values too (a device round trip)."""
    assert positions.dtype == torch.int32 and positions.is_cuda and positions.is_contiguous(), \
        "positions are a contiguous int32 device tensor"
    assert positions.device == x.device, "positions live on the activations' device"
    assert positions.numel() == tokens, "one position per token of the flattened (B, T) axes"
    if _CHECK_POSITION_VALUES and tokens:
        lo, hi = int(positions.min()), int(positions.max())
        assert 0 <= lo and hi < rows, "positions must lie in [0, %d): got %d .. %d" % (rows, lo, hi)


def _rope(x: torch.Tensor, freqs: torch.Tensor, out: Optional[torch.Tensor], n_q: int, n_kv: int,
          layout: str, backward: bool, positions: Optional[torch.Tensor] = None) -> torch.Tensor:
    assert x.dim() == 4, "activations are (B, T, heads, head_dim)"
    B, T, heads, head_dim = x.shape
    if layout == "qkv":
        assert heads == n_q + 2 * n_kv, "packed QKV needs n_q + 2*n_kv heads"
    else:
        n_q, n_kv = heads, 0
    dtype = _ROPE_DTYPES.get(x.dtype)
    if dtype is None:
        raise TypeError("RoPE storage is float32, bfloat16 or float16")
    if positions is None:
        assert freqs.dtype == torch.float32 and freqs.shape == (T, head_dim)
    else:
        assert layout == "heads", "positions go with separate q / k tensors"
        assert freqs.dtype == torch.float32 and freqs.dim() == 2 and freqs.shape[1] == head_dim
        _check_positions(positions, B * T, x, freqs.shape[0])
        T = 0                                   # the sequence length is not part of the compiled text
    if out is None:
        out = x
    else:
        assert out.shape == x.shape and out.dtype == x.dtype
        if layout == "qkv" and out.data_ptr() != x.data_ptr():
            # value heads are skipped by the kernel (neither read nor written): out of place they
            # have to be carried over by a copy first
            torch.ops.sideaware.memcpy(out, x)
    kid = _kernel("rope", (max(T, 1), n_q, n_kv, head_dim, dtype, layout, backward),
                  (("positions", positions is not None),))
    _elementwise(kid, out, None, None, None, x, freqs, None, None, positions, 0, 0, 0)
    return out


def rope_forward_qkv(x, freqs, n_q: int, n_kv: int, out=None):
    """Packed (B, T, n_q + 2*n_kv, head_dim): rotates q and k heads, leaves v heads alone.
    In place unless ``out`` is given."""
    return _rope(x, freqs, out, n_q, n_kv, "qkv", False)


def rope_backward_qkv(dout, freqs, n_q: int, n_kv: int, out=None):
    return _rope(dout, freqs, out, n_q, n_kv, "qkv", True)


def rope_forward_heads(x, freqs, out=None, positions=None):
    """(B, T, heads, head_dim), every head rotated: one call per separate q or k tensor.
    ``positions``: an int32 device tensor with one table row number per token of the flattened
    (B, T) axes, for decoding steps and packed sequences (``freqs`` then has a row for every
    position that occurs); without it token t of every sequence uses row t."""
    return _rope(x, freqs, out, 0, 0, "heads", False, positions)


def rope_backward_heads(dout, freqs, out=None, positions=None):
    return _rope(dout, freqs, out, 0, 0, "heads", True, positions)


class _Segment(ctypes.Structure):
    """``sideaware_segment`` of include/sideaware.h."""
    _fields_ = [("num_bytes", ctypes.c_size_t), ("out", ctypes.c_void_p * 4), ("inp", ctypes.c_void_p * 4),
                ("sideband_memory", ctypes.c_void_p), ("sideband_value", ctypes.c_int)]


def elementwise_batch(kernel_id: int, segments) -> None:
    """One launch over several arrays of the same op.  ``segments`` is a sequence of
    ``(num_bytes, outs, ins, sideband_tensor_or_None, sideband_value)`` with ``outs`` / ``ins``
    sequences of up to four tensors (or None)."""
    arr = (_Segment * len(segments))()
    for seg, (num_bytes, outs, ins, sideband, value) in zip(arr, segments):
        seg.num_bytes = num_bytes
        for i, t in enumerate(outs):
            seg.out[i] = wrapper._check(t, "out%d" % i) or None
        for i, t in enumerate(ins):
            seg.inp[i] = wrapper._check(t, "in%d" % i) or None
        seg.sideband_memory = sideband.data_ptr() if sideband is not None else None
        seg.sideband_value = int(value)
    device, stream = wrapper._device_and_stream()
    wrapper.library().sideaware_elementwise_batch(kernel_id, len(arr), arr, device, stream)


def _rope_heads_many(tensors, freqs: torch.Tensor, backward: bool, positions: Optional[torch.Tensor] = None):
    first = tensors[0]
    assert first.dim() == 4, "activations are (B, T, heads, head_dim)"
    T, head_dim = first.shape[1], first.shape[3]
    if positions is not None:
        return _rope_many_at_positions(tensors, freqs, backward, positions, half=False)
    dtype = _ROPE_DTYPES.get(first.dtype)
    if dtype is None:
        raise TypeError("RoPE storage is float32, bfloat16 or float16")
    assert freqs.dtype == torch.float32 and tuple(freqs.shape) == (T, head_dim)
    for t in tensors:
        assert t.dim() == 4 and t.shape[1] == T and t.shape[3] == head_dim and t.dtype == first.dtype
    kid = _kernel("rope", (T, 0, 0, head_dim, dtype, "heads", backward), (("heads_at_launch", True),))
    elementwise_batch(kid, [(t.numel() * t.element_size(), [t], [t, freqs], None, t.shape[2]) for t in tensors])
    return tensors


def _rope_many_at_positions(tensors, freqs, backward: bool, positions: torch.Tensor, half: bool):
    first = tensors[0]
    B, T, head_dim = first.shape[0], first.shape[1], first.shape[3]
    dtype = _ROPE_DTYPES.get(first.dtype)
    if dtype is None:
        raise TypeError("RoPE storage is float32, bfloat16 or float16")
    assert freqs.dtype == torch.float32 and freqs.dim() == 2 and freqs.shape[1] == head_dim
    _check_positions(positions, B * T, first, freqs.shape[0])
    for t in tensors:
        assert t.dim() == 4 and t.is_contiguous() and t.shape[:2] == first.shape[:2] and t.shape[3] == head_dim \
            and t.dtype == first.dtype
    launch_time = (("heads_at_launch", True), ("positions", True))
    if half:
        kid = _kernel("rope_half", (1, 0, head_dim, dtype, backward), launch_time)
    else:
        kid = _kernel("rope", (1, 0, 0, head_dim, dtype, "heads", backward), launch_time)
    elementwise_batch(kid, [(t.numel() * t.element_size(), [t], [t, freqs], positions, t.shape[2]) for t in tensors])
    return tensors


def rope_forward_heads_many(tensors, freqs, positions=None):
    """Rotates several (B, T, heads, head_dim) tensors in place in ONE launch: q and k of a
    grouped-query model (different head counts, same T, head_dim and dtype) share a grid.
    ``positions`` as in :func:`rope_forward_heads`."""
    return _rope_heads_many(list(tensors), freqs, False, positions)


def rope_backward_heads_many(tensors, freqs, positions=None):
    return _rope_heads_many(list(tensors), freqs, True, positions)


def _rope_half(x: torch.Tensor, freqs: torch.Tensor, out: Optional[torch.Tensor], heads_first: bool,
               backward: bool, positions: Optional[torch.Tensor] = None) -> torch.Tensor:
    assert x.dim() == 4 and x.is_contiguous(), "activations are contiguous (B, T, heads, head_dim) or (B, heads, T, head_dim)"
    if heads_first:
        _, heads, T, head_dim = x.shape
    else:
        _, T, heads, head_dim = x.shape
    dtype = _ROPE_DTYPES.get(x.dtype)
    if dtype is None:
        raise TypeError("RoPE storage is float32, bfloat16 or float16")
    if positions is None:
        assert freqs.dtype == torch.float32 and tuple(freqs.shape) == (T, head_dim)
    else:
        assert not heads_first, "positions are per token of a (B, T, heads, head_dim) tensor"
        assert freqs.dtype == torch.float32 and freqs.dim() == 2 and freqs.shape[1] == head_dim
        _check_positions(positions, x.shape[0] * T, x, freqs.shape[0])
        T = 1                                   # the sequence length is not part of the compiled text
    if out is None:
        out = x
    assert out.shape == x.shape and out.dtype == x.dtype and out.is_contiguous()
    kid = _kernel("rope_half", (T, heads, head_dim, dtype, backward, heads_first), (("positions", positions is not None),))
    _elementwise(kid, out, None, None, None, x, freqs, None, None, positions, 0, 0, 0)
    return out


def rope_half_forward(x, freqs, out=None, heads_first: bool = False, positions=None):
    """RoPE for the half-split pair layout (element i of a head pairs with element
    i + head_dim/2, the "rotate_half" convention): (B, T, heads, head_dim), or
    (B, heads, T, head_dim) with ``heads_first``.  ``freqs`` is the same (T, head_dim) table the
    interleaved ops take ([t, 2i] = cos, [t, 2i+1] = sin of pair i).  In place unless ``out`` is given.
    ``positions`` as in :func:`rope_forward_heads`."""
    return _rope_half(x, freqs, out, heads_first, False, positions)


def rope_half_backward(dout, freqs, out=None, heads_first: bool = False, positions=None):
    return _rope_half(dout, freqs, out, heads_first, True, positions)


def rope_half_forward_many(tensors, freqs, backward: bool = False, positions=None):
    """Half-split RoPE of several (B, T, heads, head_dim) tensors in place in ONE launch (q and k
    of a grouped-query model).  ``positions`` as in :func:`rope_forward_heads`."""
    tensors = list(tensors)
    if positions is not None:
        return _rope_many_at_positions(tensors, freqs, backward, positions, half=True)
    first = tensors[0]
    T, head_dim = first.shape[1], first.shape[3]
    dtype = _ROPE_DTYPES.get(first.dtype)
    if dtype is None:
        raise TypeError("RoPE storage is float32, bfloat16 or float16")
    assert freqs.dtype == torch.float32 and tuple(freqs.shape) == (T, head_dim)
    for t in tensors:
        assert t.dim() == 4 and t.is_contiguous() and t.shape[1] == T and t.shape[3] == head_dim and t.dtype == first.dtype
    kid = _kernel("rope_half", (T, 0, head_dim, dtype, backward), (("heads_at_launch", True),))
    elementwise_batch(kid, [(t.numel() * t.element_size(), [t], [t, freqs], None, t.shape[2]) for t in tensors])
    return tensors


def scale_bias_bf16(x: torch.Tensor, scale_bias: torch.Tensor, out: Optional[torch.Tensor] = None):
    """bf16 ``y = x*scale + bias`` in fp32, rounded to nearest even.  ``scale_bias`` is a device
    tensor of two fp32 values, read by the kernel, so changing them costs no compile."""
    assert x.dtype == torch.bfloat16 and scale_bias.dtype == torch.float32 and scale_bias.numel() >= 2
    if out is None:
        out = torch.empty_like(x)
    kid = _kernel("scale_bias_bf16")
    _elementwise(kid, out, None, None, None, x, None, None, None, scale_bias, 0, 0, 0)
    return out


def mxfp8_quantize(x: torch.Tensor, q: Optional[torch.Tensor] = None, scales: Optional[torch.Tensor] = None):
    """bf16 -> MXFP8: returns (E4M3 bytes as a uint8 tensor shaped like x, E8M0 scale bytes, one
    per 32 consecutive elements).  ``x.numel()`` must be a multiple of 32."""
    assert x.dtype == torch.bfloat16 and x.is_contiguous() and x.numel() % 32 == 0
    if q is None:
        q = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    if scales is None:
        scales = torch.empty(x.numel() // 32, dtype=torch.uint8, device=x.device)
    assert q.dtype == torch.uint8 and q.numel() == x.numel() and scales.numel() == x.numel() // 32
    kid = _kernel("mxfp8_quantize")
    device, stream = wrapper._device_and_stream()
    # num_bytes is the byte length of the wider array, the bf16 input, which the custom-op wrapper
    # cannot know (it sizes the launch from out0, as the reference's does): call the C entry point.
    # the sideband value is the number of 16-byte vectors: the op gathers a wave's 16 scale bytes
    # into one store wherever the whole wave lies inside the array
    wrapper.library().sideaware_elementwise(kid, x.numel() * 2, q.data_ptr(), 0, 0, 0, x.data_ptr(), 0, 0, 0,
                                            scales.data_ptr(), min(x.numel() // 8, 2 ** 31 - 1), 0, 0, device, stream)
    return q, scales


def mxfp8_dequantize(q: torch.Tensor, scales: torch.Tensor, out: Optional[torch.Tensor] = None):
    """MXFP8 -> bf16: ``q`` E4M3 bytes (uint8), ``scales`` one E8M0 byte per 32 elements."""
    assert q.dtype == torch.uint8 and scales.dtype == torch.uint8 and q.is_contiguous() and scales.is_contiguous()
    assert q.numel() % 32 == 0 and scales.numel() == q.numel() // 32
    if out is None:
        out = torch.empty(q.shape, dtype=torch.bfloat16, device=q.device)
    assert out.dtype == torch.bfloat16 and out.numel() == q.numel()
    kid = _kernel("mxfp8_dequantize")
    # out0 is the wider array, so the custom op's own sizing (from out0) is the right one
    _elementwise(kid, out, None, None, None, q, None, None, None, scales, 0, 0, 0)
    return out


def fill_int32(out: torch.Tensor, value: int):
    """Writes a 32-bit pattern over ``out`` (byte size a multiple of 16): an output-only op."""
    kid = _kernel("fill")
    _elementwise(kid, out, None, None, None, None, None, None, None, None, int(value), 0, 0)
    return out
