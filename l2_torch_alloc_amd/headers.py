"""Op headers for the run-time compiled elementwise kernel.

An op header is the text the caller hands to ``sideaware_create_kernel``: element types
``o0..o3`` / ``i0..i3``, ``reverse_order``, ``input_evict`` and ``elementwise_op``, plus optional
hooks.  The contract is the reference's (``sideaware.cu:33-48``, ``kernel_rope.cuh:1-60``,
``test.py:191-216``); the generators below bake the problem shape into the text the way the
reference's RoPE header does with its ``constexpr int T / n_head / head_dim``
(``kernel_rope.cuh:21-27``), but for any shape, for bf16 or fp16 storage and for separate q / k tensors.

Arithmetic follows the llm.c formula (``example_llmc_rope.cu:70-81``, ``kernel_rope.cuh:29-40``):
``out = (x_re*c - x_im*s, x_re*s + x_im*c)`` in fp32, each product rounded before the add (the
library compiles with contraction off), so fp32 results are bit-identical to a CPU that does not
fuse.  bf16 and fp16 storage widen exactly, compute in fp32 and round to nearest even on store.
"""
from __future__ import annotations

_UNUSED = "struct unused {};\n"


def _evict(flags) -> str:
    flags = list(flags) + [False] * (4 - len(flags))
    return "constexpr bool input_evict[4] = {%s};\n" % ", ".join("true" if f else "false" for f in flags)


def memcpy_header() -> bytes:
    """The built-in copy (kernel id 0), spelled out: 4-byte elements, input read once."""
    return (
        "#define KERNEL_NAME sideaware_copy_spelled_out\n"
        "typedef int o0;\ntypedef int i0;\n" + _UNUSED +
        "typedef unused o1, o2, o3, i1, i2, i3;\n"
        "constexpr bool reverse_order = false;\n" + _evict([True]) +
        "__device__ void elementwise_op(size_t element_idx, int sideband,\n"
        "                               o0 &out0, o1 &out1, o2 &out2, o3 &out3,\n"
        "                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {\n"
        "    out0 = in0;\n}\n"
    ).encode()


_ROPE_TYPES = {
    # storage dtype -> (declarations, element type of one (re, im) pair, widen, narrow)
    "fp32": ("", "float2", "%s", "%s"),
    "bf16": ("struct sa_bf16_pair { __bf16 x, y; };\n", "sa_bf16_pair", "(float)%s", "(__bf16)(%s)"),
    "fp16": ("struct sa_fp16_pair { _Float16 x, y; };\n", "sa_fp16_pair", "(float)%s", "(_Float16)(%s)"),
}


def rope_header(T: int, n_q: int, n_kv: int, head_dim: int, dtype: str = "fp32",
                layout: str = "qkv", backward: bool = False, unrolled: int | None = 1,
                reverse_order: bool = False, evict_input: bool = True,
                stream_input: bool | None = None, stream_output: bool | None = None,
                heads_at_launch: bool = False, positions: bool = False) -> bytes:
    """RoPE forward (or backward) in place or out of place.

    layout "qkv":   one tensor (B, T, n_q + 2*n_kv, head_dim); q and k heads are rotated, the
                    trailing n_kv value heads are skipped (neither read nor written), which is
                    the reference's packed layout (``kernel_rope.cuh:42-60``) with GQA head counts.
    layout "heads": one tensor (B, T, n_q, head_dim), every head rotated (``n_kv`` ignored):
                    separate q and k tensors take one launch each.

    in0/out0 is the activation, in1 the fp32 table (T, head_dim/2, 2) of (cos, sin) pairs.
    ``num_bytes`` at launch is the byte size of the activation tensor.

    ``heads_at_launch`` (layout "heads" only): the number of heads per token is not baked into the
    text but read from the launch's ``sideband_value``, so one compiled kernel serves q and k of a
    grouped-query model and both can go out in one batched launch (``n_q`` is then ignored).

    ``positions`` (layout "heads" only): a token's table row is not its index in the sequence but
    an int32 read from the launch's sideband pointer, one per token of the flattened (B, T) axes:
    decoding steps and packed batches of sequences at arbitrary positions (``T`` then only names
    the kernel).  The table must have a row for every position that occurs.
    """
    if dtype not in _ROPE_TYPES:
        raise ValueError("dtype must be 'fp32', 'bf16' or 'fp16'")
    if layout not in ("qkv", "heads"):
        raise ValueError("layout must be 'qkv' or 'heads'")
    if head_dim % 2:
        raise ValueError("head_dim must be even")
    decl, pair, widen, narrow = _ROPE_TYPES[dtype]
    pair_bytes = 8 if dtype == "fp32" else 4
    pairs_per_vec = 16 // pair_bytes
    half = head_dim // 2
    if half % pairs_per_vec:
        raise ValueError("head_dim/2 must be a multiple of %d for %s" % (pairs_per_vec, dtype))
    if (heads_at_launch or positions) and layout != "heads":
        raise ValueError("heads_at_launch and positions need layout 'heads'")
    total_heads = n_q + 2 * n_kv if layout == "qkv" else n_q
    rotated_heads = n_q + n_kv if layout == "qkv" else n_q
    sign_a, sign_b = ("+", "-") if backward else ("-", "+")

    name = "sideaware_rope_%s_%s_%s_t%s_h%s_%d_d%d" % ("bwd" if backward else "fwd", dtype, layout,
                                                        "pos" if positions else str(T),
                                                        "N" if heads_at_launch else str(n_q),
                                                        n_kv if layout == "qkv" else 0, head_dim)
    lines = ["#define KERNEL_NAME %s\n" % name, decl]
    if stream_input is not None:
        lines.append("#define INPUT0_STREAMING %d\n" % int(stream_input))
    if stream_output is not None:
        lines.append("#define OUTPUT_STREAMING %d\n" % int(stream_output))
    lines.append("typedef %s o0;\ntypedef %s i0;\ntypedef float2 i1;\n" % (pair, pair))
    lines.append(_UNUSED + "typedef unused o1, o2, o3, i2, i3;\n")
    if unrolled is not None:
        lines.append("#define UNROLLED %d\n" % unrolled)
    lines.append("constexpr bool reverse_order = %s;\n" % ("true" if reverse_order else "false"))
    # The table is re-read by every head of a token and must stay cached.  The activations are
    # read once, with the streaming hint.
    lines.append(_evict([evict_input, False]))
    lines.append(
        "constexpr int rope_T = %d;\n"
        "constexpr int rope_half = %d;          // pairs per head\n"
        "constexpr int rope_heads = %d;         // heads per token in this tensor\n"
        "constexpr int rope_rotated = %d;       // leading heads that are rotated\n"
        % (T, half, total_heads, rotated_heads))
    lines.append(
        "__device__ __forceinline__ void elementwise_op(size_t element_idx, int sideband,\n"
        "                               o0 &out0, o1 &out1, o2 &out2, o3 &out3,\n"
        "                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {\n"
        "    const float x_re = %s, x_im = %s;\n"
        "    const float c = in1.x, s = in1.y;\n"
        "    const float y_re = x_re * c %s x_im * s;\n"
        "    const float y_im = x_im * c %s x_re * s;\n"
        "    out0.x = %s;\n"
        "    out0.y = %s;\n"
        "}\n" % (widen % "in0.x", widen % "in0.y", sign_a, sign_b, narrow % "y_re", narrow % "y_im"))
    # A 16-byte vector holds pairs_per_vec consecutive pairs of one head of one token, so one
    # decode serves the whole vector: the table row of the token, at the head-local pair.
    if heads_at_launch or positions:
        # every head is rotated; the only thing the head count decides is where a token's row ends
        heads_expr = "(size_type)val" if heads_at_launch else "(size_type)rope_heads"
        token_expr = "mem[row]" if positions else "(int)(row % rope_T)"
        lines.append(
            "#define CUSTOM_IDX_FUNC\n"
            "__device__ __forceinline__ bool indexing(size_type vec_idx, int vec_size,\n"
            "                         size_type &idx_i0, size_type &idx_i1,\n"
            "                         size_type &idx_i2, size_type &idx_i3, int* mem, int val) {\n"
            "    const size_type pair = vec_idx * vec_size;\n"
            "    const size_type row = (pair / rope_half) / %s;      // the token, counted over batch and sequence\n"
            "    const int token = %s;\n"
            "    const int local = (int)(pair %% rope_half);\n"
            "    idx_i0 = vec_idx;\n"
            "    idx_i1 = (size_type)(((size_type)token * rope_half + local) / vec_size);\n"
            "    idx_i2 = 0;\n"
            "    idx_i3 = 0;\n"
            "    return false;\n"
            "}\n" % (heads_expr, token_expr))
        return "".join(lines).encode()
    lines.append(
        "#define CUSTOM_IDX_FUNC\n"
        "__device__ __forceinline__ bool indexing(size_type vec_idx, int vec_size,\n"
        "                         size_type &idx_i0, size_type &idx_i1,\n"
        "                         size_type &idx_i2, size_type &idx_i3, int* mem, int val) {\n"
        "    const size_type pair = vec_idx * vec_size;\n"
        "    const int head = (int)((pair / rope_half) % rope_heads);\n"
        "    const int token = (int)((pair / ((size_type)rope_heads * rope_half)) % rope_T);\n"
        "    const int local = (int)(pair % rope_half);\n"
        "    idx_i0 = vec_idx;\n"
        "    idx_i1 = (size_type)((token * rope_half + local) / vec_size);\n"
        "    idx_i2 = 0;\n"
        "    idx_i3 = 0;\n"
        "    return head >= rope_rotated;\n"
        "}\n")
    return "".join(lines).encode()


_ROPE_HALF_TYPES = {
    # storage dtype -> (element type, elements per 16-byte vector)
    "fp32": ("float", 4),
    "bf16": ("__bf16", 8),
    "fp16": ("_Float16", 8),
}


def rope_half_header(T: int, n_heads: int, head_dim: int, dtype: str = "bf16", backward: bool = False,
                     heads_first: bool = False, heads_at_launch: bool = False, unrolled: int | None = 1,
                     evict_input: bool = True, positions: bool = False) -> bytes:
    """RoPE for the half-split pair layout ("rotate_half": element i of a head is paired with
    element i + head_dim/2, as Hugging Face / GPT-NeoX style models store q and k), forward or
    backward, in place or out of place.

    The reference's op (``kernel_rope.cuh:29-60``) pairs neighbouring elements (2i, 2i+1), so a
    lane holds both halves of every pair it rotates.  Here the partner of a lane's 16-byte vector
    lies head_dim/2 elements further on (or back), in the vector of a lane ``head_dim/2 /
    vec_size`` lanes away in the same wave: the op is a ``CUSTOM_VECTOR_OP`` that fetches the
    partner's vector with a lane exchange, the kind of op the reference's ``vector_op`` hook
    exists for (``sideaware.cu:81-83``).  The arithmetic per pair is the same as the interleaved
    op's: ``(x1*c - x2*s, x2*c + x1*s)`` in fp32, each product rounded before the add, so the
    result equals the interleaved op on the permuted head bit for bit.

    in0/out0: the activation, (B, T, heads, head_dim), or (B, heads, T, head_dim) with
    ``heads_first``; in1: the same fp32 table as :func:`rope_header` takes, (T, head_dim/2, 2) of
    (cos, sin).  With ``heads_at_launch`` the head count is read from ``sideband_value``; with
    ``positions`` a token's table row is an int32 read from the sideband pointer, one per token
    of the flattened (B, T) axes, as in :func:`rope_header`.
    head_dim/2 must be a power-of-two number of 16-byte vectors (bf16 / fp16: head_dim = 16, 32,
    64, 128, 256, 512; fp32: 8 ... 256), so that a head never straddles a 64-lane wave.
    """
    if dtype not in _ROPE_HALF_TYPES:
        raise ValueError("dtype must be 'fp32', 'bf16' or 'fp16'")
    elem, vec = _ROPE_HALF_TYPES[dtype]
    half = head_dim // 2
    lanes = half // vec                                  # lanes between a vector and its partner
    if head_dim % 2 or half % vec or lanes < 1 or lanes > 32 or lanes & (lanes - 1):
        raise ValueError("head_dim/2 must be a power-of-two multiple (1..32) of %d elements for %s" % (vec, dtype))
    if heads_at_launch and heads_first:
        raise ValueError("with heads_first the head count is not needed: leave heads_at_launch off")
    if positions and heads_first:
        raise ValueError("positions are per token of a (B, T, heads, head_dim) tensor")
    name = "sideaware_rope_half_%s_%s_%s_t%s_h%s_d%d" % (
        "bwd" if backward else "fwd", dtype, "bhtd" if heads_first else "bthd", "pos" if positions else str(T),
        "N" if heads_at_launch else str(n_heads), head_dim)
    heads_expr = "(size_type)val" if heads_at_launch else "rope_heads"
    if heads_first:
        token = "(int)(row % rope_T)"
    elif positions:
        token = "mem[row / %s]" % heads_expr
    else:
        token = "(int)((row / %s) %% rope_T)" % heads_expr
    # forward: first half x1*c - x2*s, second half x2*c + x1*s; backward: the signs swap
    keep_sign, send_sign = ("-", "+") if backward else ("+", "-")
    lines = ["#define KERNEL_NAME %s\n" % name,
             # the table is read as plain floats: a lane loads vec_size of them, the (cos, sin) of
             # the vec_size/2 pairs it rotates
             "typedef %s o0;\ntypedef %s i0;\ntypedef float i1;\n" % (elem, elem),
             _UNUSED + "typedef unused o1, o2, o3, i2, i3;\n"]
    if unrolled is not None:
        lines.append("#define UNROLLED %d\n" % unrolled)
    lines.append("constexpr bool reverse_order = false;\n" + _evict([evict_input, False]))
    lines.append(
        "constexpr int rope_T = %d;\n"
        "constexpr int rope_dim = %d;           // elements per head\n"
        "constexpr int rope_half = %d;          // pairs per head\n"
        "constexpr int rope_heads = %d;         // heads per token\n"
        "constexpr int rope_partner_lanes = %d; // lanes between the two halves of a pair\n"
        "constexpr int rope_vec = %d;           // elements per 16-byte vector\n"
        % (T, head_dim, half, max(n_heads, 1), lanes, vec))
    lines.append(
        "__device__ __forceinline__ void elementwise_op(size_t element_idx, int sideband,\n"
        "                               o0 &out0, o1 &out1, o2 &out2, o3 &out3,\n"
        "                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {}\n"
        "// A lane holds rope_vec elements of one half of a head; the lane rope_partner_lanes away holds\n"
        "// the same positions of the other half.  The two split the work by position, not by half: the\n"
        "// lane of the first half rotates the first rope_vec/2 pairs, its partner the rest, so each\n"
        "// needs only the table entries of its own pairs.  They trade the elements the other needs\n"
        "// before the rotation and the results the other stores after it: four 32-bit lane exchanges\n"
        "// per 16-byte vector in all.\n"
        "// One 32-bit word of the partner lane.  Distances of 1, 2 and 8 lanes are data-parallel\n"
        "// moves inside a row of 16 lanes, 16 and 32 lanes are gfx950's row and half-wave swaps: all\n"
        "// run in the vector ALU.  4 lanes goes through the LDS crossbar.  `upper` says whether this\n"
        "// lane is the one with the higher number of the two.\n"
        "__device__ __forceinline__ int rope_partner_word(int v, bool upper) {\n"
        "    if constexpr (rope_partner_lanes == 1) return __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, false);      // quad_perm:[1,0,3,2]\n"
        "    else if constexpr (rope_partner_lanes == 2) return __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xf, 0xf, false); // quad_perm:[2,3,0,1]\n"
        "    else if constexpr (rope_partner_lanes == 8) return __builtin_amdgcn_update_dpp(0, v, 0x128, 0xf, 0xf, false); // row_ror:8\n"
        "    else if constexpr (rope_partner_lanes == 16) {\n"
        "        const auto r = __builtin_amdgcn_permlane16_swap((unsigned)v, (unsigned)v, false, false);\n"
        "        return (int)(upper ? r[0] : r[1]);\n"
        "    } else if constexpr (rope_partner_lanes == 32) {\n"
        "        const auto r = __builtin_amdgcn_permlane32_swap((unsigned)v, (unsigned)v, false, false);\n"
        "        return (int)(upper ? r[0] : r[1]);\n"
        "    } else return __shfl_xor(v, rope_partner_lanes);\n"
        "}\n"
        "#define CUSTOM_IDX_FUNC\n"
        "__device__ __forceinline__ bool indexing(size_type vec_idx, int vec_size,\n"
        "                         size_type &idx_i0, size_type &idx_i1,\n"
        "                         size_type &idx_i2, size_type &idx_i3, int* mem, int val) {\n"
        "    const size_type elem = vec_idx * vec_size;\n"
        "    const size_type row = elem / rope_dim;                 // (batch, token, head) or (batch, head, token)\n"
        "    const int token = %s;\n"
        "    const int in_head = (int)(elem %% rope_dim);\n"
        "    const bool second = in_head >= rope_half;\n"
        "    const int pair = (second ? in_head - rope_half + rope_vec / 2 : in_head);   // first pair this lane rotates\n"
        "    idx_i0 = vec_idx;\n"
        "    idx_i1 = (size_type)(((size_type)token * rope_half + pair) / (rope_vec / 2));   // in units of rope_vec floats\n"
        "    idx_i2 = 0;\n"
        "    idx_i3 = 0;\n"
        "    return false;\n"
        "}\n"
        "#define CUSTOM_VECTOR_OP\n"
        "__device__ __forceinline__ void vector_op(size_type vec_idx, int vec_size,\n"
        "                          o0 *out0, o1 *out1, o2 *out2, o3 *out3,\n"
        "                          const i0 *in0, const i1 *in1, const i2 *in2, const i3 *in3,\n"
        "                          int* sideband_memory, int sideband_value) {\n"
        "    constexpr int H = rope_vec / 2;                        // pairs per lane\n"
        "    constexpr int W = H * (int)sizeof(i0) / 4;             // 32-bit words in half a vector\n"
        "    const bool second = (int)((vec_idx * vec_size) %% rope_dim) >= rope_half;\n"
        "    // The lane of the first half keeps its lower H elements and gives away the upper H; the lane\n"
        "    // of the second half the other way round.\n"
        "    int words[2 * W], mine_w[W], offer[W], got[W];\n"
        "    __builtin_memcpy(words, in0, 8 * W);\n"
        "    #pragma unroll\n"
        "    for (int w = 0; w < W; w++) {\n"
        "        mine_w[w] = second ? words[W + w] : words[w];\n"
        "        offer[w] = second ? words[w] : words[W + w];\n"
        "    }\n"
        "    #pragma unroll\n"
        "    for (int w = 0; w < W; w++) got[w] = rope_partner_word(offer[w], second);\n"
        "    i0 mine[H], theirs[H], keep[H], send[H];\n"
        "    __builtin_memcpy(mine, mine_w, 4 * W);\n"
        "    __builtin_memcpy(theirs, got, 4 * W);\n"
        "    // With m this lane's element of a pair and t the partner's, the first-half lane keeps\n"
        "    // y1 = m*c - t*s and sends y2 = t*c + m*s; the second-half lane keeps y2 = m*c + t*s and\n"
        "    // sends y1 = t*c - m*s (backward: the signs swap).  One expression serves both: the sign of\n"
        "    // the s-products is flipped in the first-half lane, which is exact.\n"
        "    const unsigned flip = second ? 0u : 0x80000000u;\n"
        "    #pragma unroll\n"
        "    for (int i = 0; i < H; i++) {\n"
        "        const float m = (float)mine[i], t = (float)theirs[i];\n"
        "        const float c = in1[2 * i], s = in1[2 * i + 1];\n"
        "        const float ts = __uint_as_float(__float_as_uint(t * s) ^ flip);\n"
        "        const float ms = __uint_as_float(__float_as_uint(m * s) ^ flip);\n"
        "        keep[i] = (o0)(m * c %s ts);\n"
        "        send[i] = (o0)(t * c %s ms);\n"
        "    }\n"
        "    __builtin_memcpy(offer, send, 4 * W);\n"
        "    #pragma unroll\n"
        "    for (int w = 0; w < W; w++) got[w] = rope_partner_word(offer[w], second);\n"
        "    __builtin_memcpy(mine_w, keep, 4 * W);\n"
        "    #pragma unroll\n"
        "    for (int w = 0; w < W; w++) {\n"
        "        words[w] = second ? got[w] : mine_w[w];\n"
        "        words[W + w] = second ? mine_w[w] : got[w];\n"
        "    }\n"
        "    __builtin_memcpy(out0, words, 8 * W);\n"
        "}\n" % (token, keep_sign, send_sign))
    return "".join(lines).encode()


def scale_bias_bf16_header(unrolled: int | None = None, evict_input: bool = True) -> bytes:
    """bf16 ``y = x*scale + bias``; scale and bias are two fp32 values read from the sideband
    pointer at launch, so one compiled kernel serves every (scale, bias)."""
    lines = ["#define KERNEL_NAME sideaware_scale_bias_bf16\n",
             "typedef __bf16 o0;\ntypedef __bf16 i0;\n", _UNUSED, "typedef unused o1, o2, o3, i1, i2, i3;\n"]
    if unrolled is not None:
        lines.append("#define UNROLLED %d\n" % unrolled)
    lines.append("constexpr bool reverse_order = false;\n" + _evict([evict_input]))
    lines.append(
        "__device__ __forceinline__ void elementwise_op(size_t element_idx, int sideband,\n"
        "                               o0 &out0, o1 &out1, o2 &out2, o3 &out3,\n"
        "                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {}\n"
        "#define CUSTOM_VECTOR_OP\n"
        "__device__ __forceinline__ void vector_op(size_type vec_idx, int vec_size,\n"
        "                          o0 *out0, o1 *out1, o2 *out2, o3 *out3,\n"
        "                          const i0 *in0, const i1 *in1, const i2 *in2, const i3 *in3,\n"
        "                          int* sideband_memory, int sideband_value) {\n"
        "    const float scale = ((const float*)sideband_memory)[0];\n"
        "    const float bias  = ((const float*)sideband_memory)[1];\n"
        "    #pragma unroll\n"
        "    for (int i = 0; i < vec_size; i++) {\n"
        "        const float p = (float)in0[i] * scale;\n"
        "        out0[i] = (__bf16)(p + bias);\n"
        "    }\n"
        "}\n")
    return "".join(lines).encode()


def mxfp8_quantize_header(unrolled: int | None = 1) -> bytes:
    """bf16 -> MXFP8 (OCP Microscaling: E4M3 elements with one E8M0 scale byte per 32 elements).

    The op the reference cites as the reason for its ``vector_op`` hook and sideband pointer
    (``sideaware.cu:81-83``): the maximum magnitude of 32 consecutive elements is needed before any
    of them can be converted.  A 16-byte vector holds 8 bf16 elements, so a block is 4 neighbouring
    lanes, and the maximum travels between them with two lane exchanges.  in0 = bf16 input,
    out0 = E4M3 bytes, the sideband pointer receives the scale bytes (element count / 32 of them).
    The element count must be a multiple of 32 so that no block is cut by the end of the array.

    shared_exp = floor(log2(max|x|)) - 8, clamped to [-127, 127] (an all-zero block gets -127);
    scale byte = shared_exp + 127; element = E4M3(x * 2^-shared_exp), round to nearest even,
    saturated at +-448.  Finite inputs.
    """
    lines = ["#define KERNEL_NAME sideaware_mxfp8_quantize\n",
             "typedef unsigned char o0;\ntypedef __bf16 i0;\n", _UNUSED,
             "typedef unused o1, o2, o3, i1, i2, i3;\n"]
    if unrolled is not None:
        lines.append("#define UNROLLED %d\n" % unrolled)
    lines.append("constexpr bool reverse_order = false;\n" + _evict([True]))
    lines.append(
        "__device__ __forceinline__ void elementwise_op(size_t element_idx, int sideband,\n"
        "                               o0 &out0, o1 &out1, o2 &out2, o3 &out3,\n"
        "                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {}\n"
        "#define CUSTOM_VECTOR_OP\n"
        "__device__ __forceinline__ void vector_op(size_type vec_idx, int vec_size,\n"
        "                          o0 *out0, o1 *out1, o2 *out2, o3 *out3,\n"
        "                          const i0 *in0, const i1 *in1, const i2 *in2, const i3 *in3,\n"
        "                          int* sideband_memory, int sideband_value) {\n"
        "    float v[8];\n"
        "    float amax = 0.0f;\n"
        "    #pragma unroll\n"
        "    for (int i = 0; i < 8; i++) { v[i] = (float)in0[i]; amax = fmaxf(amax, fabsf(v[i])); }\n"
        "    // a block of 32 elements is 4 neighbouring lanes: lanes 4k..4k+3 of the wave\n"
        "    // (data-parallel moves inside each group of four lanes: quad_perm [1,0,3,2], then [2,3,0,1])\n"
        "    amax = fmaxf(amax, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(amax), 0xB1, 0xf, 0xf, false)));\n"
        "    amax = fmaxf(amax, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(amax), 0x4E, 0xf, 0xf, false)));\n"
        "    // floor(log2(amax)) is the exponent field of the float (a bf16 subnormal widens to an\n"
        "    // fp32 subnormal with field 0, far below the clamp anyway)\n"
        "    int shared_exp = (int)((__float_as_uint(amax) >> 23) & 0xff) - 127 - 8;\n"
        "    if (amax == 0.0f || shared_exp < -127) shared_exp = -127;\n"
        "    if (shared_exp > 127) shared_exp = 127;\n"
        "    // The scale bytes.  A wave's 64 vectors are 16 blocks, 16 consecutive scale bytes: when the\n"
        "    // whole wave lies inside the array (the launch passes the number of vectors as the sideband\n"
        "    // value) the bytes of a row of 16 lanes are gathered into one word with row shifts, the four\n"
        "    // rows' words are read across, and lane 0 writes all 16 bytes with one store, written through\n"
        "    // the private L2 like the outputs; elsewhere (the last, partial wave; a launch that does not\n"
        "    // pass the count) every fourth lane stores its own byte.\n"
        "    const unsigned int sb = (unsigned int)(shared_exp + 127);\n"
        "    unsigned char *scales = (unsigned char*)sideband_memory;\n"
        "#if defined(__AMDGCN__)\n"
        "    if (((vec_idx | 63) < (size_type)sideband_value) && (((size_t)scales & 15) == 0)) {\n"
        "        unsigned int word = sb;\n"
        "        word |= (unsigned int)__builtin_amdgcn_update_dpp(0, (int)sb, 0x104, 0xf, 0xf, false) << 8;    // row_shl:4\n"
        "        word |= (unsigned int)__builtin_amdgcn_update_dpp(0, (int)sb, 0x108, 0xf, 0xf, false) << 16;   // row_shl:8\n"
        "        word |= (unsigned int)__builtin_amdgcn_update_dpp(0, (int)sb, 0x10C, 0xf, 0xf, false) << 24;   // row_shl:12\n"
        "        typedef int sa_scale_v4 __attribute__((ext_vector_type(4)));\n"
        "        sa_scale_v4 all;\n"
        "        all.x = __builtin_amdgcn_readlane((int)word, 0);\n"
        "        all.y = __builtin_amdgcn_readlane((int)word, 16);\n"
        "        all.z = __builtin_amdgcn_readlane((int)word, 32);\n"
        "        all.w = __builtin_amdgcn_readlane((int)word, 48);\n"
        "        if ((vec_idx & 63) == 0) {\n"
        "            sa_scale_v4 *dst = (sa_scale_v4*)(scales + (vec_idx >> 2));\n"
        "            asm volatile(\"global_store_dwordx4 %0, %1, off sc1\\n\\ts_nop 1\" : : \"v\"(dst), \"v\"(all) : \"memory\");\n"
        "        }\n"
        "    } else\n"
        "#endif\n"
        "    if ((vec_idx & 3) == 0) scales[vec_idx >> 2] = (unsigned char)sb;\n"
        "    // two conversions fill one 32-bit word with four E4M3 bytes: the second writes the upper half\n"
        "    int words[2] = {0, 0};\n"
        "    #pragma unroll\n"
        "    for (int i = 0; i < 8; i += 2) {\n"
        "        // ldexpf scales exactly over the whole range (2^127 and 2^-127 are not both normal floats)\n"
        "        float a = ldexpf(v[i], -shared_exp), b = ldexpf(v[i + 1], -shared_exp);\n"
        "        a = __builtin_amdgcn_fmed3f(a, -448.0f, 448.0f);\n"
        "        b = __builtin_amdgcn_fmed3f(b, -448.0f, 448.0f);\n"
        "        words[i / 4] = (i & 2) ? __builtin_amdgcn_cvt_pk_fp8_f32(a, b, words[i / 4], true)\n"
        "                               : __builtin_amdgcn_cvt_pk_fp8_f32(a, b, words[i / 4], false);\n"
        "    }\n"
        "    __builtin_memcpy(out0, words, 8);\n"
        "}\n")
    return "".join(lines).encode()


def mxfp8_dequantize_header(unrolled: int | None = None) -> bytes:
    """MXFP8 -> bf16: the inverse of :func:`mxfp8_quantize_header`.  in0 = E4M3 bytes, the
    sideband pointer holds the E8M0 scale bytes (one per 32 elements), out0 = bf16
    ``element * 2^(scale - 127)``, which is exact: an E4M3 element has four significant bits.
    A 16-byte output vector holds 8 elements, so four neighbouring vectors share a scale byte.
    """
    lines = ["#define KERNEL_NAME sideaware_mxfp8_dequantize\n",
             "typedef __bf16 o0;\ntypedef unsigned char i0;\n", _UNUSED,
             "typedef unused o1, o2, o3, i1, i2, i3;\n"]
    if unrolled is not None:
        lines.append("#define UNROLLED %d\n" % unrolled)
    lines.append("constexpr bool reverse_order = false;\n" + _evict([True]))
    lines.append(
        "__device__ __forceinline__ void elementwise_op(size_t element_idx, int sideband,\n"
        "                               o0 &out0, o1 &out1, o2 &out2, o3 &out3,\n"
        "                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {}\n"
        "#define CUSTOM_VECTOR_OP\n"
        "__device__ __forceinline__ void vector_op(size_type vec_idx, int vec_size,\n"
        "                          o0 *out0, o1 *out1, o2 *out2, o3 *out3,\n"
        "                          const i0 *in0, const i1 *in1, const i2 *in2, const i3 *in3,\n"
        "                          int* sideband_memory, int sideband_value) {\n"
        "    const int shared_exp = (int)((const unsigned char*)sideband_memory)[vec_idx >> 2] - 127;\n"
        "    #pragma unroll\n"
        "    for (int i = 0; i < 8; i += 4) {\n"
        "        int packed;\n"
        "        __builtin_memcpy(&packed, in0 + i, 4);\n"
        "        out0[i + 0] = (__bf16)ldexpf(__builtin_amdgcn_cvt_f32_fp8(packed, 0), shared_exp);\n"
        "        out0[i + 1] = (__bf16)ldexpf(__builtin_amdgcn_cvt_f32_fp8(packed, 1), shared_exp);\n"
        "        out0[i + 2] = (__bf16)ldexpf(__builtin_amdgcn_cvt_f32_fp8(packed, 2), shared_exp);\n"
        "        out0[i + 3] = (__bf16)ldexpf(__builtin_amdgcn_cvt_f32_fp8(packed, 3), shared_exp);\n"
        "    }\n"
        "}\n")
    return "".join(lines).encode()


def fill_header() -> bytes:
    """Writes the 32-bit sideband value to every element: an output-only op (no in0)."""
    return (
        "#define KERNEL_NAME sideaware_fill_int32\n"
        "typedef int o0;\n" + _UNUSED + "typedef unused o1, o2, o3, i0, i1, i2, i3;\n"
        "constexpr bool reverse_order = false;\n" + _evict([]) +
        "__device__ void elementwise_op(size_t element_idx, int sideband,\n"
        "                               o0 &out0, o1 &out1, o2 &out2, o3 &out3,\n"
        "                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {\n"
        "    out0 = sideband;\n}\n"
    ).encode()
