/*
 * CPU oracle for the sideaware elementwise hot path: llm.c RoPE (table, forward,
 * backward), the bf16 in-place variant, bf16 scale+bias and byte copy.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or calls
 * this file; only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg
 * may use it, and there only as the checker.
 *
 * It restates, in plain C, the arithmetic of the reference's CPU functions:
 *   precompute_freqs_cis       example_llmc_rope.cu:19-52
 *   apply_rotary_emb_forward   example_llmc_rope.cu:54-86
 *   apply_rotary_emb_backward  example_llmc_rope.cu:166-195
 * and the per-pair op and index decode of the reference's device header
 *   elementwise_op / indexing  kernel_rope.cuh:29-60
 * generalised from (n_head, n_head, n_head) packed QKV to (Nq, Nkv, Nkv) heads and to
 * separate q / k tensors, which is what the Llama-3 shaped workload needs.
 *
 * Build with -ffp-contract=off: every product is rounded to fp32 before the add or
 * subtract, exactly as the reference's scalar C does on a CPU without FMA
 * contraction.  The GPU kernels are compiled the same way, so fp32 results are
 * expected to be bit-identical, not merely close.
 *
 * How each function is pinned (tests/test_oracle.py):
 *   oracle_freqs_cis        closed forms: i=0 => (cos t, sin t); t=0 => (1,0); float64
 *                           recomputation; Llama-3.1 scaling on its three wavelength
 *                           regimes by hand-picked frequencies
 *   oracle_rope_*           numpy complex64 multiply; t=0 identity; per-pair norm;
 *                           V heads bit-identical; hand-computed (B=1,T=2,NH=1,HS=4);
 *                           backward(forward(x)) == x up to rounding
 *   oracle_f32_to_bf16      torch.Tensor.to(torch.bfloat16) on CPU, all 2^16 high
 *                           halves x several low halves, NaN/Inf included
 *   oracle_scale_bias_bf16  torch CPU fp32 multiply, add, .to(bfloat16)
 *   oracle_f32_to_e4m3      torch.Tensor.to(torch.float8_e4m3fn) on CPU over every in-range value
 *                           on a fine grid and every midpoint between neighbouring E4M3 values
 *   oracle_mxfp8_quantize   closed forms (power-of-two blocks, zero block, the scale of a block
 *                           whose maximum sits just below / at a power of two), the error bound
 *                           of the format, and quantize(dequantize(quantize(x))) == quantize(x)
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#ifndef M_PI
#define M_PI 3.14159265358979323846
#endif

/* ---- bf16 <-> fp32 -------------------------------------------------------------- */

/* IEEE round-to-nearest-even fp32 -> bf16; NaN stays NaN (quiet bit forced). */
uint16_t oracle_f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        return (uint16_t)((u >> 16) | 0x0040u);
    }
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

float oracle_bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

void oracle_f32_to_bf16_array(uint16_t *out, const float *in, size_t n) {
    for (size_t i = 0; i < n; i++) out[i] = oracle_f32_to_bf16(in[i]);
}

void oracle_bf16_to_f32_array(float *out, const uint16_t *in, size_t n) {
    for (size_t i = 0; i < n; i++) out[i] = oracle_bf16_to_f32(in[i]);
}

/* ---- frequency table (example_llmc_rope.cu:19-52) ----------------------------------- */

/* freqs_cis is (end, dim) fp32: [t*dim + 2i] = cos(t*f_i), [t*dim + 2i + 1] = sin(t*f_i),
 * f_i = 1 / theta^(2i/dim), optionally rescaled the Llama-3.1 way (:25-43). */
void oracle_freqs_cis(float *freqs_cis, int dim, int end, float theta, int use_scaled) {
    for (int i = 0; i < dim / 2; i++) {
        float freq = 1.0f / powf(theta, (float)(2 * i) / dim);
        if (use_scaled) {
            const int scale_factor = 8;
            const int low_freq_factor = 1;
            const int high_freq_factor = 4;
            const int old_context_len = 8192;
            const float low_freq_wavelen = (float)old_context_len / low_freq_factor;
            const float high_freq_wavelen = (float)old_context_len / high_freq_factor;
            /* the reference multiplies a float by the double constant M_PI and
             * divides in double before narrowing (:32) */
            float wavelen = 2.0f * M_PI / freq;
            if (wavelen < high_freq_wavelen) {
                /* high frequency: unchanged */
            } else if (wavelen > low_freq_wavelen) {
                freq /= scale_factor;
            } else {
                float smooth = ((float)old_context_len / wavelen - low_freq_factor) /
                               (high_freq_factor - low_freq_factor);
                freq = (1.0f - smooth) * freq / scale_factor + smooth * freq;
            }
        }
        for (int t = 0; t < end; t++) {
            float angle = (float)t * freq;
            freqs_cis[(size_t)t * dim + 2 * i] = cosf(angle);
            freqs_cis[(size_t)t * dim + 2 * i + 1] = sinf(angle);
        }
    }
}

/* ---- the per-pair op (kernel_rope.cuh:29-40, example_llmc_rope.cu:70-81) ------------ */

static inline void rotate(float *o_re, float *o_im, float x_re, float x_im, float c, float s) {
    *o_re = x_re * c - x_im * s;
    *o_im = x_re * s + x_im * c;
}

/* ---- packed QKV forward, fp32 (example_llmc_rope.cu:54-86 generalised to Nq/Nkv) ---- */

/* inp/out: (B, T, Nq + 2*Nkv, head_dim) fp32 row-major; q heads then k heads are rotated,
 * the trailing Nkv value heads are copied.  Nq == Nkv == n_head is the reference's case. */
void oracle_rope_forward_qkv_f32(float *out, const float *inp, const float *freqs_cis,
                                 int B, int T, int Nq, int Nkv, int head_dim) {
    const int N = Nq + 2 * Nkv;
    for (int b = 0; b < B; b++) {
        for (int t = 0; t < T; t++) {
            size_t idx_bt = ((size_t)b * T + t) * (size_t)N * head_dim;
            for (int h = 0; h < N; h++) {
                size_t idx_bth = idx_bt + (size_t)h * head_dim;
                if (h >= Nq + Nkv) {
                    for (int d = 0; d < head_dim; d++) out[idx_bth + d] = inp[idx_bth + d];
                    continue;
                }
                for (int d = 0; d < head_dim / 2; d++) {
                    size_t idx = idx_bth + 2 * (size_t)d;
                    size_t fidx = (size_t)t * head_dim + 2 * (size_t)d;
                    float re, im;
                    rotate(&re, &im, inp[idx], inp[idx + 1], freqs_cis[fidx], freqs_cis[fidx + 1]);
                    out[idx] = re;
                    out[idx + 1] = im;
                }
            }
        }
    }
}

/* Backward of the above (example_llmc_rope.cu:166-195): conjugate rotation, accumulated
 * into dinp (which the reference zero-fills first); value heads pass straight through. */
void oracle_rope_backward_qkv_f32(float *dinp, const float *dout, const float *freqs_cis,
                                  int B, int T, int Nq, int Nkv, int head_dim) {
    const int N = Nq + 2 * Nkv;
    for (int b = 0; b < B; b++) {
        for (int t = 0; t < T; t++) {
            size_t idx_bt = ((size_t)b * T + t) * (size_t)N * head_dim;
            for (int h = 0; h < N; h++) {
                size_t idx_bth = idx_bt + (size_t)h * head_dim;
                if (h >= Nq + Nkv) {
                    for (int d = 0; d < head_dim; d++) dinp[idx_bth + d] = dout[idx_bth + d];
                    continue;
                }
                for (int d = 0; d < head_dim / 2; d++) {
                    size_t idx = idx_bth + 2 * (size_t)d;
                    size_t fidx = (size_t)t * head_dim + 2 * (size_t)d;
                    float c = freqs_cis[fidx], s = freqs_cis[fidx + 1];
                    dinp[idx] += dout[idx] * c + dout[idx + 1] * s;
                    dinp[idx + 1] += -dout[idx] * s + dout[idx + 1] * c;
                }
            }
        }
    }
}

/* ---- one tensor of heads, (B, T, NH, head_dim): every head rotated ------------------ */

void oracle_rope_forward_heads_f32(float *out, const float *inp, const float *freqs_cis,
                                   int B, int T, int NH, int head_dim) {
    for (int b = 0; b < B; b++) {
        for (int t = 0; t < T; t++) {
            for (int h = 0; h < NH; h++) {
                size_t base = (((size_t)b * T + t) * NH + h) * (size_t)head_dim;
                for (int d = 0; d < head_dim / 2; d++) {
                    size_t idx = base + 2 * (size_t)d;
                    size_t fidx = (size_t)t * head_dim + 2 * (size_t)d;
                    float re, im;
                    rotate(&re, &im, inp[idx], inp[idx + 1], freqs_cis[fidx], freqs_cis[fidx + 1]);
                    out[idx] = re;
                    out[idx + 1] = im;
                }
            }
        }
    }
}

/* Same, bf16 storage: load bf16, widen, rotate in fp32, round to nearest even, store.
 * out may alias inp (the in-place workload). */
void oracle_rope_forward_heads_bf16(uint16_t *out, const uint16_t *inp, const float *freqs_cis,
                                    int B, int T, int NH, int head_dim) {
    for (int b = 0; b < B; b++) {
        for (int t = 0; t < T; t++) {
            for (int h = 0; h < NH; h++) {
                size_t base = (((size_t)b * T + t) * NH + h) * (size_t)head_dim;
                for (int d = 0; d < head_dim / 2; d++) {
                    size_t idx = base + 2 * (size_t)d;
                    size_t fidx = (size_t)t * head_dim + 2 * (size_t)d;
                    float re, im;
                    rotate(&re, &im, oracle_bf16_to_f32(inp[idx]), oracle_bf16_to_f32(inp[idx + 1]),
                           freqs_cis[fidx], freqs_cis[fidx + 1]);
                    out[idx] = oracle_f32_to_bf16(re);
                    out[idx + 1] = oracle_f32_to_bf16(im);
                }
            }
        }
    }
}

/* Conjugate rotation in place of the forward one: the backward of a single head tensor,
 * written (not accumulated), as the reference's in-place backward kernel does
 * (example_llmc_rope.cu:197-228). */
void oracle_rope_backward_heads_f32(float *dinp, const float *dout, const float *freqs_cis,
                                    int B, int T, int NH, int head_dim) {
    for (int b = 0; b < B; b++) {
        for (int t = 0; t < T; t++) {
            for (int h = 0; h < NH; h++) {
                size_t base = (((size_t)b * T + t) * NH + h) * (size_t)head_dim;
                for (int d = 0; d < head_dim / 2; d++) {
                    size_t idx = base + 2 * (size_t)d;
                    size_t fidx = (size_t)t * head_dim + 2 * (size_t)d;
                    float c = freqs_cis[fidx], s = freqs_cis[fidx + 1];
                    float re = dout[idx], im = dout[idx + 1];
                    dinp[idx] = re * c + im * s;
                    dinp[idx + 1] = -re * s + im * c;
                }
            }
        }
    }
}

/* ---- bf16 y = x*scale + bias: widen, multiply (rounded), add (rounded), RNE ---------- */

void oracle_scale_bias_bf16(uint16_t *y, const uint16_t *x, float scale, float bias, size_t n) {
    for (size_t i = 0; i < n; i++) {
        float p = oracle_bf16_to_f32(x[i]) * scale;
        float r = p + bias;
        y[i] = oracle_f32_to_bf16(r);
    }
}

/* ---- bf16 -> MXFP8 (OCP Microscaling v1.0: E4M3 elements, one E8M0 scale per 32) -------- */

/* The reference names this op as the reason its template has a vector_op hook and a sideband
 * pointer ("BF16 -> MXFP8 with microscaling where we need the absmax over 32 elements",
 * sideaware.cu:81-83) but ships no implementation; this follows the OCP MX specification:
 *   shared_exp = floor(log2(max|x|)) - 8        (8 = exponent of the largest E4M3 binade)
 *   scale byte = clamp(shared_exp, -127, 127) + 127, an all-zero block gets scale byte 0
 *   element    = E4M3( x * 2^-shared_exp ), round to nearest even, saturating at +-448
 * Finite inputs only. */

/* fp32 -> E4M3 (4 exponent bits, bias 7, 3 mantissa bits, no infinities, 0x7f/0xff = NaN),
 * round to nearest even, saturating: |v| > 448 -> 448. */
uint8_t oracle_f32_to_e4m3(float v) {
    uint32_t u;
    memcpy(&u, &v, 4);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80);
    float a = fabsf(v);
    if (a != a) return (uint8_t)(sign | 0x7f);
    if (a >= 448.0f) return (uint8_t)(sign | 0x7e);
    int e;
    float m = frexpf(a, &e);                       /* a = m * 2^e, m in [0.5, 1) */
    int exp = e - 1;                               /* a = (2m) * 2^exp, 2m in [1, 2) */
    if (a == 0.0f || exp < -6) {                   /* zero and subnormals: quantum 2^-9 */
        int k = (int)nearbyintf(a * 512.0f);       /* default rounding mode: nearest even; 0..8 */
        return (uint8_t)(sign | k);                /* 8 is the encoding of the smallest normal */
    }
    float q = (2.0f * m) * 8.0f;                   /* in [8, 16): mantissa with 3 fraction bits */
    int k = (int)nearbyintf(q);                    /* 8..16 */
    if (k == 16) { k = 8; exp += 1; }
    if (exp > 8 || (exp == 8 && k > 14)) return (uint8_t)(sign | 0x7e);
    return (uint8_t)(sign | ((exp + 7) << 3) | (k - 8));
}

float oracle_e4m3_to_f32(uint8_t b) {
    int sign = b & 0x80, e = (b >> 3) & 0xf, m = b & 7;
    float v;
    if (e == 0xf && m == 7) v = NAN;
    else if (e == 0) v = ldexpf((float)m, -9);
    else v = ldexpf((float)(8 + m), e - 7 - 3);
    return sign ? -v : v;
}

/* x: n bf16 bit patterns, n a multiple of 32.  q: n E4M3 bytes.  scales: n/32 E8M0 bytes. */
void oracle_mxfp8_quantize(uint8_t *q, uint8_t *scales, const uint16_t *x, size_t n) {
    for (size_t b = 0; b < n / 32; b++) {
        float amax = 0.0f;
        for (int i = 0; i < 32; i++) {
            float a = fabsf(oracle_bf16_to_f32(x[b * 32 + i]));
            if (a > amax) amax = a;
        }
        int shared_exp = -127;
        if (amax > 0.0f) {
            int e;
            (void)frexpf(amax, &e);                /* amax = m * 2^e, m in [0.5,1): floor(log2) = e - 1 */
            shared_exp = (e - 1) - 8;
            if (shared_exp < -127) shared_exp = -127;
            if (shared_exp > 127) shared_exp = 127;
        }
        scales[b] = (uint8_t)(shared_exp + 127);
        for (int i = 0; i < 32; i++) {
            float v = ldexpf(oracle_bf16_to_f32(x[b * 32 + i]), -shared_exp);
            q[b * 32 + i] = oracle_f32_to_e4m3(v);
        }
    }
}

/* bf16( E4M3 element * 2^(scale - 127) ): exact, an element has 4 significant bits. */
void oracle_mxfp8_dequantize(uint16_t *x, const uint8_t *q, const uint8_t *scales, size_t n) {
    for (size_t i = 0; i < n; i++) {
        float v = ldexpf(oracle_e4m3_to_f32(q[i]), (int)scales[i / 32] - 127);
        x[i] = oracle_f32_to_bf16(v);
    }
}

/* ---- byte copy: the memcpy kernel's whole contract is dst == src --------------------- */

void oracle_memcpy(void *dst, const void *src, size_t n) { memcpy(dst, src, n); }

/* ---- llm.c tolerance rule (example_llmc_common.h:313-351), fp32 build ----------------- */

/* Returns the number of elements with |ref - got| > tol + |ref| * FLT_EPSILON, skipping
 * non-finite reference values, the way validate_result counts faults. */
size_t oracle_validate_f32(const float *got, const float *ref, size_t n, float tolerance) {
    const float epsilon = 1.1920928955078125e-07f;
    size_t faults = 0;
    for (size_t i = 0; i < n; i++) {
        if (!isfinite(ref[i])) continue;
        float t_eff = tolerance + fabsf(ref[i]) * epsilon;
        if (fabsf(ref[i] - got[i]) > t_eff) faults++;
    }
    return faults;
}
