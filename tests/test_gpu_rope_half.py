"""GPU parity of the half-split ("rotate_half") RoPE op against the CPU oracle, bit for bit.

The op exchanges 16-byte vectors between lanes of a wave, so the cases cover every lane distance
(1 ... 32 lanes between the halves of a pair), all three storage types, both tensor layouts,
backward, arrays that end in a partial tile, out of place, several tensors in one launch, and the
Llama-3-8B q and k at full size.
"""
import numpy as np
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu


def bits(t: torch.Tensor) -> np.ndarray:
    t = t.detach().contiguous().cpu()
    view = {2: torch.int16, 4: torch.int32}[t.element_size()]
    return t.view(view).numpy().view({2: np.uint16, 4: np.uint32}[t.element_size()])


def assert_no_library_error(sa):
    assert sa.sideaware_last_error() == "", sa.sideaware_last_error()


@pytest.mark.parametrize("B,T,H,D", [(1, 8, 1, 8), (2, 33, 3, 16), (1, 64, 5, 32), (2, 40, 7, 64), (1, 130, 3, 128),
                                     (2, 16, 2, 256)])
def test_fp32_forward_and_backward_vs_oracle(sa, B, T, H, D):
    from l2_torch_alloc_amd import ops
    g = torch.Generator().manual_seed(B * 1000 + T + D)
    x = torch.randn(B, T, H, D, generator=g)
    table = O.freqs_cis(D, T, 10000.0)
    freqs = torch.from_numpy(table).cuda()
    y = ops.rope_half_forward(x.cuda(), freqs)
    torch.cuda.synchronize()
    assert_no_library_error(sa)
    want = O.rope_half_forward_heads_f32(x.numpy(), table)
    assert np.array_equal(bits(y), want.view(np.uint32))
    # backward, out of place, from the forward result
    dx = torch.empty_like(y)
    ops.rope_half_backward(y, freqs, out=dx)
    torch.cuda.synchronize()
    assert np.array_equal(bits(dx), O.rope_half_backward_heads_f32(want, table).view(np.uint32))
    assert np.array_equal(bits(y), want.view(np.uint32))             # the input of an out-of-place launch is untouched


@pytest.mark.parametrize("B,T,H,D", [(1, 8, 2, 16), (2, 33, 3, 32), (3, 40, 5, 64), (2, 100, 9, 128), (1, 24, 2, 512)])
def test_bf16_vs_oracle_both_layouts(sa, B, T, H, D):
    from l2_torch_alloc_amd import ops
    g = torch.Generator().manual_seed(7 * T + D)
    x = torch.randn(B, T, H, D, generator=g).to(torch.bfloat16)
    table = O.freqs_cis(D, T, 500000.0)
    freqs = torch.from_numpy(table).cuda()
    want = O.rope_half_forward_heads_bf16(bits(x), table)
    y = ops.rope_half_forward(x.cuda(), freqs)
    torch.cuda.synchronize()
    assert_no_library_error(sa)
    assert np.array_equal(bits(y), want)
    # (B, heads, T, D): the same numbers, transposed
    xt = x.transpose(1, 2).contiguous()
    yt = ops.rope_half_forward(xt.cuda(), freqs, heads_first=True)
    torch.cuda.synchronize()
    assert_no_library_error(sa)
    assert np.array_equal(bits(yt), np.ascontiguousarray(np.swapaxes(want, 1, 2)))
    assert np.array_equal(bits(yt), O.rope_half_forward_heads_bf16(bits(xt), table, heads_first=True))


def test_fp16_vs_the_oracles_fp32_result_narrowed_by_numpy(sa):
    from l2_torch_alloc_amd import ops
    B, T, H, D = 2, 50, 3, 64
    x = torch.randn(B, T, H, D, generator=torch.Generator().manual_seed(5)).to(torch.float16)
    table = O.freqs_cis(D, T, 10000.0)
    y = ops.rope_half_forward(x.cuda(), torch.from_numpy(table).cuda())
    torch.cuda.synchronize()
    assert_no_library_error(sa)
    want = O.rope_half_forward_heads_f32(x.float().numpy(), table).astype(np.float16)
    assert np.array_equal(bits(y), want.view(np.uint16))


def test_q_and_k_in_one_launch_at_llama3_size_vs_oracle(sa):
    from l2_torch_alloc_amd import ops
    B, T, D = 8, 4096, 128
    table = O.freqs_cis(D, T, 500000.0)
    freqs = torch.from_numpy(table).cuda()
    g = torch.Generator().manual_seed(12)
    q_h = torch.randn(B, T, 32, D, generator=g).to(torch.bfloat16)
    k_h = torch.randn(B, T, 8, D, generator=g).to(torch.bfloat16)
    q, k = q_h.cuda(), k_h.cuda()
    ops.rope_half_forward_many([q, k], freqs)
    torch.cuda.synchronize()
    assert_no_library_error(sa)
    assert np.array_equal(bits(k), O.rope_half_forward_heads_bf16(bits(k_h), table))
    # q: the first and the last batch entries against the oracle, all of it against the one-tensor launch
    want0 = O.rope_half_forward_heads_bf16(bits(q_h[:1]), table)
    want7 = O.rope_half_forward_heads_bf16(bits(q_h[7:]), table)
    got = bits(q)
    assert np.array_equal(got[:1], want0) and np.array_equal(got[7:], want7)
    q2 = ops.rope_half_forward(q_h.cuda(), freqs)
    torch.cuda.synchronize()
    assert np.array_equal(bits(q2), got)
    # backward of both in one launch brings the inputs back to within rounding
    ops.rope_half_forward_many([q, k], freqs, backward=True)
    torch.cuda.synchronize()
    assert_no_library_error(sa)
    assert float((q.float().cpu() - q_h.float()).abs().max()) <= 0.0625


def test_batched_launches_replay_from_a_hip_graph(sa):
    # the batched launch carries its segment table in the kernel arguments (no device memory is
    # written by the call), so it is captured like any kernel: q and k of both pair layouts
    from l2_torch_alloc_amd import ops
    T, D = 96, 128
    table = O.freqs_cis(D, T, 500000.0)
    freqs = torch.from_numpy(table).cuda()
    g = torch.Generator().manual_seed(21)
    q0 = torch.randn(2, T, 8, D, generator=g).to(torch.bfloat16)
    k0 = torch.randn(2, T, 2, D, generator=g).to(torch.bfloat16)
    q, k, q2, k2 = q0.cuda(), k0.cuda(), q0.cuda(), k0.cuda()
    ops.rope_half_forward_many([q.clone(), k.clone()], freqs)          # compiled outside the capture
    ops.rope_forward_heads_many([q2.clone(), k2.clone()], freqs)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            ops.rope_half_forward_many([q, k], freqs)
            ops.rope_forward_heads_many([q2, k2], freqs)
    torch.cuda.current_stream().wait_stream(side)
    want_q, want_k = O.rope_half_forward_heads_bf16(bits(q0), table), O.rope_half_forward_heads_bf16(bits(k0), table)
    want_q2, want_k2 = O.rope_forward_heads_bf16(bits(q0), table), O.rope_forward_heads_bf16(bits(k0), table)
    for trial in range(3):
        for dst, src in ((q, q0), (k, k0), (q2, q0), (k2, k0)):
            dst.copy_(src)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(bits(q), want_q) and np.array_equal(bits(k), want_k), trial
        assert np.array_equal(bits(q2), want_q2) and np.array_equal(bits(k2), want_k2), trial
    assert_no_library_error(sa)


# --------------------------------------------------------------------------------------- positions

def _rows(table, positions):
    """The table a flattened (1, B*T, heads, D) run of the oracle needs: row i = the row of token i."""
    return np.ascontiguousarray(table[positions.reshape(-1)])


@pytest.mark.parametrize("B,T,H,D", [(3, 5, 4, 64), (16, 1, 32, 128), (2, 129, 3, 128)])
def test_rope_at_given_positions_vs_oracle_both_pair_layouts(sa, B, T, H, D):
    # decoding steps and packed sequences: each token names its own table row
    from l2_torch_alloc_amd import ops
    max_pos = 1000
    table = O.freqs_cis(D, max_pos, 500000.0)
    freqs = torch.from_numpy(table).cuda()
    g = torch.Generator().manual_seed(B * 100 + T)
    pos = torch.randint(0, max_pos, (B, T), generator=g, dtype=torch.int32)
    x = torch.randn(B, T, H, D, generator=g).to(torch.bfloat16)
    flat = bits(x).reshape(1, B * T, H, D)
    rows = _rows(table, pos.numpy())
    want_pairs = O.rope_forward_heads_bf16(flat, rows).reshape(B, T, H, D)
    want_half = O.rope_half_forward_heads_bf16(flat, rows).reshape(B, T, H, D)
    pos_d = pos.cuda()
    y = ops.rope_forward_heads(x.cuda(), freqs, positions=pos_d)
    z = ops.rope_half_forward(x.cuda(), freqs, positions=pos_d)
    torch.cuda.synchronize()
    assert_no_library_error(sa)
    assert np.array_equal(bits(y), want_pairs)
    assert np.array_equal(bits(z), want_half)
    # positions 0..T-1 in every sequence are the plain op
    plain = torch.arange(T, dtype=torch.int32).repeat(B, 1).cuda()
    if T <= max_pos:
        a = ops.rope_forward_heads(x.cuda(), freqs, positions=plain)
        b = ops.rope_forward_heads(x.cuda(), freqs[:T].contiguous())
        torch.cuda.synchronize()
        assert np.array_equal(bits(a), bits(b))


def test_q_and_k_at_given_positions_in_one_launch_and_backward(sa):
    from l2_torch_alloc_amd import ops
    B, T, D, max_pos = 4, 7, 128, 300
    table = O.freqs_cis(D, max_pos, 10000.0)
    freqs = torch.from_numpy(table).cuda()
    g = torch.Generator().manual_seed(77)
    pos = torch.randint(0, max_pos, (B, T), generator=g, dtype=torch.int32)
    rows = _rows(table, pos.numpy())
    q0 = torch.randn(B, T, 8, D, generator=g)
    k0 = torch.randn(B, T, 2, D, generator=g)
    for half in (False, True):
        q, k = q0.cuda(), k0.cuda()
        fwd = O.rope_half_forward_heads_f32 if half else O.rope_forward_heads_f32
        bwd = O.rope_half_backward_heads_f32 if half else O.rope_backward_heads_f32
        if half:
            ops.rope_half_forward_many([q, k], freqs, positions=pos.cuda())
        else:
            ops.rope_forward_heads_many([q, k], freqs, positions=pos.cuda())
        torch.cuda.synchronize()
        assert_no_library_error(sa)
        want_q = fwd(q0.numpy().reshape(1, B * T, 8, D), rows)
        want_k = fwd(k0.numpy().reshape(1, B * T, 2, D), rows)
        assert np.array_equal(bits(q).reshape(want_q.shape), want_q.view(np.uint32))
        assert np.array_equal(bits(k).reshape(want_k.shape), want_k.view(np.uint32))
        if half:
            ops.rope_half_forward_many([q, k], freqs, backward=True, positions=pos.cuda())
        else:
            ops.rope_backward_heads_many([q, k], freqs, positions=pos.cuda())
        torch.cuda.synchronize()
        assert np.array_equal(bits(q).reshape(want_q.shape), bwd(want_q, rows).view(np.uint32))
        assert np.array_equal(bits(k).reshape(want_k.shape), bwd(want_k, rows).view(np.uint32))


def test_committed_golden_vectors(sa):
    import os
    from l2_torch_alloc_amd import ops
    golden = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    g = np.load(os.path.join(golden, "rope_half_fp32_heads.npz"))
    freqs = torch.from_numpy(g["freqs"]).cuda()
    y = ops.rope_half_forward(torch.from_numpy(g["x"]).cuda(), freqs)
    dx = ops.rope_half_backward(y.clone(), freqs)
    torch.cuda.synchronize()
    assert np.array_equal(bits(y), g["y"].view(np.uint32)) and np.array_equal(bits(dx), g["dx"].view(np.uint32))
    g = np.load(os.path.join(golden, "rope_half_bf16_heads_llama3.npz"))
    x = torch.from_numpy(g["x"].view(np.int16).copy()).view(torch.bfloat16).cuda()
    y = ops.rope_half_forward(x, torch.from_numpy(g["freqs"]).cuda())
    torch.cuda.synchronize()
    assert_no_library_error(sa)
    assert np.array_equal(bits(y), g["y"])
