"""Pins the CPU oracle against what the mathematics fixes, independently of its own code.

Reference being restated: example_llmc_rope.cu:19-86, :166-195; kernel_rope.cuh:29-60.
None of these checks re-types the oracle's loops: they use numpy complex arithmetic,
float64 recomputation, closed forms, torch's own bf16 rounding, and a case worked by hand.
"""
import math

import numpy as np
import pytest
import torch

from oracle import oracle as O


def rng(seed):
    return np.random.default_rng(seed)


# ---------------------------------------------------------------- frequency table

@pytest.mark.parametrize("theta", [10000.0, 500000.0])
@pytest.mark.parametrize("dim,end", [(8, 5), (64, 33), (128, 17)])
def test_freqs_closed_forms(theta, dim, end):
    f = O.freqs_cis(dim, end, theta)
    assert f.shape == (end, dim) and f.dtype == np.float32
    # t = 0: angle 0 for every pair
    assert np.all(f[0, 0::2] == 1.0) and np.all(f[0, 1::2] == 0.0)
    # i = 0: frequency exactly 1, so the first pair is (cos t, sin t) of the fp32 t
    t = np.arange(end, dtype=np.float32)
    np.testing.assert_allclose(f[:, 0], np.cos(t.astype(np.float64)), atol=1e-7)
    np.testing.assert_allclose(f[:, 1], np.sin(t.astype(np.float64)), atol=1e-7)
    # unit modulus everywhere
    np.testing.assert_allclose(f[:, 0::2] ** 2 + f[:, 1::2] ** 2, 1.0, atol=3e-7)


def test_freqs_float64_recompute():
    dim, end, theta = 128, 64, 500000.0
    f = O.freqs_cis(dim, end, theta)
    i = np.arange(dim // 2, dtype=np.float64)
    # the fp32 exponent 2i/dim and fp32 pow, then fp32 t*freq, limit how close float64 gets
    freq = (1.0 / np.power(np.float32(theta), (2 * i / dim).astype(np.float32))).astype(np.float32)
    ang = (np.arange(end, dtype=np.float32)[:, None] * freq[None, :]).astype(np.float32)
    # numpy's fp32 power and libm's powf may differ by an ulp of freq; at row t that moves
    # the angle by t * freq * 2^-23, so the bound grows with t
    tol = 1e-6 + np.arange(end, dtype=np.float64)[:, None] * 2.5e-7
    assert np.all(np.abs(f[:, 0::2] - np.cos(ang.astype(np.float64))) <= tol)
    assert np.all(np.abs(f[:, 1::2] - np.sin(ang.astype(np.float64))) <= tol)


def test_freqs_llama31_scaling_regimes():
    # Llama-3.1 rule: wavelength < 2048 keeps the frequency, > 8192 divides it by 8, and in
    # between blends linearly in (8192/wavelen - 1)/3.  Recover the per-pair frequency from
    # the t=1 row and compare with the unscaled one.
    dim, theta = 128, 500000.0
    plain = O.freqs_cis(dim, 2, theta, use_scaled=False)
    scaled = O.freqs_cis(dim, 2, theta, use_scaled=True)
    f_plain = np.arctan2(plain[1, 1::2].astype(np.float64), plain[1, 0::2].astype(np.float64))
    f_scaled = np.arctan2(scaled[1, 1::2].astype(np.float64), scaled[1, 0::2].astype(np.float64))
    wavelen = 2 * math.pi / f_plain
    hi = wavelen < 2048
    lo = wavelen > 8192
    mid = ~hi & ~lo
    assert hi.any() and lo.any() and mid.any(), "all three regimes must be exercised"
    np.testing.assert_allclose(f_scaled[hi], f_plain[hi], rtol=1e-6)
    np.testing.assert_allclose(f_scaled[lo], f_plain[lo] / 8, rtol=1e-5, atol=1e-9)
    smooth = (8192 / wavelen[mid] - 1) / 3
    np.testing.assert_allclose(f_scaled[mid], (1 - smooth) * f_plain[mid] / 8 + smooth * f_plain[mid],
                               rtol=2e-5)


# ---------------------------------------------------------------- rotation

def _complex_rope(x, f):
    """x (..., T, H, HS) fp32, f (T, HS): rotate with numpy complex128 arithmetic."""
    xc = x[..., 0::2].astype(np.float64) + 1j * x[..., 1::2].astype(np.float64)
    fc = f[:, 0::2].astype(np.float64) + 1j * f[:, 1::2].astype(np.float64)
    yc = xc * fc[:, None, :]
    out = np.empty(x.shape, dtype=np.float64)
    out[..., 0::2] = yc.real
    out[..., 1::2] = yc.imag
    return out


def test_rope_hand_worked():
    # B=1, T=2, one q head + one k head + one v head, head_dim 4, theta=10000 =>
    # pair frequencies 1 and 1/100.  Row t=0 is untouched; row t=1 rotates pair 0 by 1 rad
    # and pair 1 by 0.01 rad.
    f = O.freqs_cis(4, 2, 10000.0)
    x = np.zeros((1, 2, 3, 4), dtype=np.float32)
    x[0, :, 0] = [1, 0, 0, 2]       # q: (1+0j), (0+2j)
    x[0, :, 1] = [3, 4, -1, 1]      # k
    x[0, :, 2] = [9, 8, 7, 6]       # v
    y = O.rope_forward_qkv_f32(x, f, 1, 1)
    np.testing.assert_array_equal(y[0, 0], x[0, 0])
    c1, s1, c2, s2 = math.cos(1), math.sin(1), math.cos(0.01), math.sin(0.01)
    np.testing.assert_allclose(y[0, 1, 0], [c1, s1, -2 * s2, 2 * c2], rtol=1e-6)
    np.testing.assert_allclose(y[0, 1, 1], [3 * c1 - 4 * s1, 3 * s1 + 4 * c1, -c2 - s2, -s2 + c2],
                               rtol=1e-6)
    np.testing.assert_array_equal(y[0, 1, 2], x[0, 1, 2])


@pytest.mark.parametrize("B,T,Nq,Nkv,HS", [(2, 7, 3, 3, 8), (1, 16, 8, 2, 64), (2, 5, 4, 1, 128)])
def test_rope_qkv_vs_complex(B, T, Nq, Nkv, HS):
    x = rng(B * T).standard_normal((B, T, Nq + 2 * Nkv, HS)).astype(np.float32)
    f = O.freqs_cis(HS, T, 10000.0)
    y = O.rope_forward_qkv_f32(x, f, Nq, Nkv)
    ref = _complex_rope(x, f)
    qk = Nq + Nkv
    np.testing.assert_allclose(y[:, :, :qk], ref[:, :, :qk], atol=1e-6, rtol=1e-6)
    # value heads: bit-identical copy
    assert np.array_equal(y[:, :, qk:].view(np.uint32), x[:, :, qk:].view(np.uint32))
    # token 0 is the identity, bit for bit
    assert np.array_equal(y[:, 0].view(np.uint32), x[:, 0].view(np.uint32))
    # rotation preserves each pair's modulus
    n_in = x[:, :, :qk, 0::2].astype(np.float64) ** 2 + x[:, :, :qk, 1::2].astype(np.float64) ** 2
    n_out = y[:, :, :qk, 0::2].astype(np.float64) ** 2 + y[:, :, :qk, 1::2].astype(np.float64) ** 2
    np.testing.assert_allclose(n_out, n_in, rtol=2e-6, atol=1e-9)


def test_rope_heads_matches_qkv_slices():
    # The separate-tensor form must agree bit for bit with the q and k slices of packed QKV.
    B, T, Nq, Nkv, HS = 2, 9, 4, 2, 16
    x = rng(3).standard_normal((B, T, Nq + 2 * Nkv, HS)).astype(np.float32)
    f = O.freqs_cis(HS, T, 500000.0)
    y = O.rope_forward_qkv_f32(x, f, Nq, Nkv)
    yq = O.rope_forward_heads_f32(np.ascontiguousarray(x[:, :, :Nq]), f)
    yk = O.rope_forward_heads_f32(np.ascontiguousarray(x[:, :, Nq:Nq + Nkv]), f)
    assert np.array_equal(yq, y[:, :, :Nq]) and np.array_equal(yk, y[:, :, Nq:Nq + Nkv])


def test_rope_backward_inverts_forward():
    B, T, Nq, Nkv, HS = 2, 11, 2, 2, 32
    x = rng(5).standard_normal((B, T, Nq + 2 * Nkv, HS)).astype(np.float32)
    f = O.freqs_cis(HS, T, 10000.0)
    y = O.rope_forward_qkv_f32(x, f, Nq, Nkv)
    back = O.rope_backward_qkv_f32(y, f, Nq, Nkv)   # conjugate rotation of a unit phasor
    np.testing.assert_allclose(back, x, atol=2e-6, rtol=2e-6)
    # and against the complex conjugate product directly
    conj = f.copy()
    conj[:, 1::2] *= -1
    ref = _complex_rope(y, conj)
    np.testing.assert_allclose(back[:, :, :Nq + Nkv], ref[:, :, :Nq + Nkv], atol=1e-6, rtol=1e-6)
    bh = O.rope_backward_heads_f32(np.ascontiguousarray(y[:, :, :Nq]), f)
    assert np.array_equal(bh, back[:, :, :Nq])


# ---------------------------------------------------------------- bf16

def test_bf16_rne_matches_torch_exhaustively():
    # every 16-bit high half combined with low halves that straddle the rounding boundary
    hi = np.arange(1 << 16, dtype=np.uint32) << 16
    lows = np.array([0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF], dtype=np.uint32)
    bits = (hi[:, None] | lows[None, :]).reshape(-1)
    x = bits.view(np.float32)
    got = O.f32_to_bf16(x)
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    # NaN payloads may differ between implementations; they must stay NaN
    assert np.all(np.isnan(O.bf16_to_f32(got[nan])))


def test_bf16_widen_is_exact():
    h = np.arange(1 << 16, dtype=np.uint16)
    f = O.bf16_to_f32(h)
    assert np.array_equal(f.view(np.uint32), h.astype(np.uint32) << 16)


def test_rope_bf16_vs_torch_rounding():
    B, T, NH, HS = 2, 6, 3, 16
    x32 = rng(7).standard_normal((B, T, NH, HS)).astype(np.float32)
    xb = O.f32_to_bf16(x32)
    f = O.freqs_cis(HS, T, 500000.0)
    got = O.rope_forward_heads_bf16(xb, f)
    # independent path: widen with torch, rotate with the fp32 oracle, round with torch
    xw = torch.from_numpy(xb.view(np.int16)).view(torch.bfloat16).to(torch.float32).numpy()
    y32 = O.rope_forward_heads_f32(xw, f)
    want = torch.from_numpy(y32).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, want)
    # in place (out aliases inp) gives the same bits
    buf = xb.copy()
    O.lib().oracle_rope_forward_heads_bf16(buf.ctypes.data, buf.ctypes.data, f.ctypes.data, B, T, NH, HS)
    assert np.array_equal(buf, want)


def test_scale_bias_bf16_vs_torch():
    x32 = rng(11).standard_normal(4096).astype(np.float32) * 3
    xb = O.f32_to_bf16(x32)
    scale, bias = 1.7, -0.3
    got = O.scale_bias_bf16(xb, scale, bias)
    t = torch.from_numpy(xb.view(np.int16)).view(torch.bfloat16).to(torch.float32)
    want = (t * torch.tensor(scale, dtype=torch.float32) + torch.tensor(bias, dtype=torch.float32))
    want = want.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, want)


def test_ulp_distance_helper():
    a = np.array([0x3F80, 0x3F80, 0x0001, 0x8001, 0x7F7F], dtype=np.uint16)
    b = np.array([0x3F81, 0x3F7F, 0x8001, 0x0000, 0x7F7F], dtype=np.uint16)
    assert O.bf16_ulp_distance(a, b).tolist() == [1, 1, 2, 1, 0]


# ---------------------------------------------------------------- misc

def test_memcpy_and_validate():
    src = rng(0).integers(0, 256, 12432, dtype=np.uint8)
    assert np.array_equal(O.memcpy(src), src)
    ref = np.array([1.0, 2.0, np.inf, 0.0], dtype=np.float32)
    got = np.array([1.0 + 5e-6, 2.1, 123.0, 2e-5], dtype=np.float32)
    assert O.validate_f32(got, ref, 1e-5) == 2      # 2.1 and 2e-5 fault; inf is skipped


# ---------------------------------------------------------------- MXFP8 (E4M3 + E8M0 per 32)

def _torch_e4m3(values: np.ndarray) -> np.ndarray:
    t = torch.from_numpy(np.asarray(values, dtype=np.float32).copy())
    return t.to(torch.float8_e4m3fn).view(torch.uint8).numpy()


def test_e4m3_decode_table():
    codes = np.arange(256, dtype=np.uint8)
    mine = O.e4m3_to_f32(codes)
    theirs = torch.from_numpy(codes.copy()).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    nan = np.isnan(theirs)
    assert np.array_equal(np.isnan(mine), nan)
    assert np.array_equal(mine[~nan], theirs[~nan])
    assert float(np.nanmax(mine)) == 448.0


def test_e4m3_encode_matches_torch_on_values_midpoints_and_a_fine_grid():
    pos = np.sort(O.e4m3_to_f32(np.arange(0, 0x7f, dtype=np.uint8)))       # every finite magnitude
    mids = (pos[:-1].astype(np.float64) + pos[1:]) / 2                       # exact ties
    eps = np.concatenate([np.nextafter(mids.astype(np.float32), np.float32(np.inf)),
                          np.nextafter(mids.astype(np.float32), np.float32(-np.inf))])
    grid = rng(1).uniform(-448, 448, 20000).astype(np.float32)
    tiny = rng(2).uniform(-0.02, 0.02, 5000).astype(np.float32)
    vals = np.concatenate([pos, -pos, mids.astype(np.float32), -mids.astype(np.float32), eps, grid, tiny])
    vals = vals[np.abs(vals) <= 448]
    assert np.array_equal(O.f32_to_e4m3(vals), _torch_e4m3(vals))
    # saturation instead of NaN beyond the largest value
    assert O.f32_to_e4m3([449.0, 1e9, -1e9]).tolist() == [0x7e, 0x7e, 0xfe]


def test_mxfp8_closed_forms():
    ones = O.f32_to_bf16(np.ones(32, dtype=np.float32))
    q, s = O.mxfp8_quantize(ones)
    # max 1 = 2^0: shared exponent 0 - 8 = -8, scale byte 119; 1 * 2^8 = 256 = 0x78 in E4M3
    assert s.tolist() == [119] and set(q.tolist()) == {0x78}
    zeros = np.zeros(32, dtype=np.uint16)
    q, s = O.mxfp8_quantize(zeros)
    assert s.tolist() == [0] and not q.any()
    # the largest element always lands in [256, 448]: just below a power of two it saturates
    blk = np.full(32, 0.25, dtype=np.float32)
    blk[5] = -1.9921875                        # bf16-exact, floor(log2) = 0 -> x * 256 = -510 -> -448
    q, s = O.mxfp8_quantize(O.f32_to_bf16(blk))
    assert s.tolist() == [119] and q[5] == 0xfe and q[0] == O.f32_to_e4m3([64.0])[0]
    blk[5] = 2.0                               # at the power of two the scale steps up
    q, s = O.mxfp8_quantize(O.f32_to_bf16(blk))
    assert s.tolist() == [120] and q[5] == 0x78 and q[0] == O.f32_to_e4m3([32.0])[0]


def test_mxfp8_error_bound_and_idempotence():
    x = (rng(3).standard_normal(32 * 512) * np.exp(rng(4).uniform(-20, 20, 32 * 512))).astype(np.float32)
    xb = O.f32_to_bf16(x)
    q, s = O.mxfp8_quantize(xb)
    back = O.bf16_to_f32(O.mxfp8_dequantize(q, s)).reshape(-1, 32).astype(np.float64)
    orig = O.bf16_to_f32(xb).reshape(-1, 32).astype(np.float64)
    scale = np.ldexp(1.0, s.astype(np.int64) - 127)[:, None]
    # within half an E4M3 step of the element's binade (2^-4 relative), or half the smallest
    # subnormal step of the block, or the saturation gap (448 vs < 512) for the block maximum
    err = np.abs(back - orig)
    bound = np.maximum(np.abs(orig) * 2.0 ** -4, scale * 2.0 ** -10)
    sat = np.abs(orig) > 448 * scale
    assert np.all(err[~sat] <= bound[~sat] * (1 + 1e-12))
    assert np.all(err[sat] <= 64 * scale.repeat(32, 1)[sat])
    # quantising the dequantised values changes nothing
    q2, s2 = O.mxfp8_quantize(O.mxfp8_dequantize(q, s))
    assert np.array_equal(q2, q) and np.array_equal(s2[s != 0], s[s != 0])


def test_fp16_narrowing_used_for_fp16_rope_is_ieee_round_to_nearest_even():
    # fp16 RoPE storage is checked on the GPU against numpy's float32 -> float16 conversion of the
    # oracle's fp32 result.  Pin that conversion: against torch's own, and against the textbook
    # rule on exact midpoints between neighbouring float16 values (ties go to the even mantissa).
    import torch
    rng = np.random.default_rng(3)
    x = np.concatenate([rng.standard_normal(200000).astype(np.float32) * 8,
                        np.array([0.0, -0.0, 65504.0, 65520.0, 1e-8, 6e-8, 6.1e-5, np.inf, -np.inf], np.float32)])
    assert np.array_equal(x.astype(np.float16).view(np.uint16),
                          torch.from_numpy(x).to(torch.float16).view(torch.int16).numpy().view(np.uint16))
    lo = np.arange(0x3c00, 0x3c00 + 64, dtype=np.uint16)              # 1.0 .. in float16 steps of 2^-10
    a, b = lo.view(np.float16).astype(np.float32), (lo + 1).view(np.float16).astype(np.float32)
    mid = (a + b) / 2                                                  # exact in float32
    got = mid.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, np.where(lo % 2 == 0, lo, lo + 1))


# ---------------------------------------------------------------- half-split pair layout

def _direct_half_rope(x, f, backward=False):
    """(x1*c - x2*s, x2*c + x1*s) written out in numpy float32: every product and sum rounded on
    its own, in the order the interleaved formula has them (example_llmc_rope.cu:70-81)."""
    h = x.shape[-1] // 2
    c = f[:, 0::2][None, :, None, :].astype(np.float32)
    s = f[:, 1::2][None, :, None, :].astype(np.float32)
    x1, x2 = x[..., :h], x[..., h:]
    if backward:
        return np.concatenate([x1 * c + x2 * s, x2 * c - x1 * s], axis=-1)
    return np.concatenate([x1 * c - x2 * s, x2 * c + x1 * s], axis=-1)


@pytest.mark.parametrize("B,T,NH,HS", [(2, 7, 3, 8), (1, 16, 8, 64), (2, 5, 4, 128)])
def test_rope_half_split_layout_vs_the_formula_written_out(B, T, NH, HS):
    x = rng(B * T + HS).standard_normal((B, T, NH, HS)).astype(np.float32)
    f = O.freqs_cis(HS, T, 10000.0)
    y = O.rope_half_forward_heads_f32(x, f)
    assert np.array_equal(y.view(np.uint32), _direct_half_rope(x, f).view(np.uint32))
    # a float64 complex product of (x1 + i x2) with (cos + i sin)
    z = (x[..., :HS // 2].astype(np.float64) + 1j * x[..., HS // 2:]) * \
        (f[:, 0::2].astype(np.float64) + 1j * f[:, 1::2])[None, :, None, :]
    np.testing.assert_allclose(y[..., :HS // 2], z.real, atol=1e-6, rtol=1e-6)
    np.testing.assert_allclose(y[..., HS // 2:], z.imag, atol=1e-6, rtol=1e-6)
    # token 0 is the identity; a dropped permutation would show as the interleaved result
    assert np.array_equal(y[:, 0].view(np.uint32), x[:, 0].view(np.uint32))
    if T > 1 and HS > 2:
        assert not np.array_equal(y, O.rope_forward_heads_f32(x, f))
    # backward: the formula written out, and the inverse of forward
    dx = O.rope_half_backward_heads_f32(y, f)
    assert np.array_equal(dx.view(np.uint32), _direct_half_rope(y, f, backward=True).view(np.uint32))
    np.testing.assert_allclose(dx, x, atol=2e-6, rtol=2e-6)
    # (B, heads, T, HS) is the same op on the transposed tensor
    xt = np.ascontiguousarray(np.swapaxes(x, 1, 2))
    assert np.array_equal(O.rope_half_forward_heads_f32(xt, f, heads_first=True), np.swapaxes(y, 1, 2))


def test_rope_half_split_bf16_vs_torch_rounding():
    B, T, NH, HS = 2, 6, 3, 32
    xb = O.f32_to_bf16(rng(9).standard_normal((B, T, NH, HS)).astype(np.float32))
    f = O.freqs_cis(HS, T, 500000.0)
    got = O.rope_half_forward_heads_bf16(xb, f)
    xw = torch.from_numpy(xb.view(np.int16)).view(torch.bfloat16).to(torch.float32).numpy()
    want = torch.from_numpy(_direct_half_rope(xw, f)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, want)
