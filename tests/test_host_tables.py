"""Host-side helpers of the Python layer that need no GPU: the cos/sin table built with torch CPU
ops against the oracle's libm version (example_llmc_rope.cu:19-52), and the op-header generators'
argument checks."""
import numpy as np
import pytest

from l2_torch_alloc_amd import headers, ops
from oracle import oracle as O


@pytest.mark.parametrize("theta,scaled", [(10000.0, False), (500000.0, False), (10000.0, True), (500000.0, True)])
@pytest.mark.parametrize("head_dim,end", [(64, 1024), (128, 4096)])
def test_torch_table_matches_the_libm_table(theta, scaled, head_dim, end):
    mine = ops.freqs_cis_table(head_dim, end, theta, scaled).numpy()
    ref = O.freqs_cis(head_dim, end, theta, scaled)
    assert mine.shape == ref.shape == (end, head_dim)
    # same formula in fp32; torch's and libm's pow/cos/sin may differ in the last place, and an ulp of
    # the frequency moves the angle at row t by t * 2^-24 relative
    t = np.arange(end, dtype=np.float64)[:, None]
    assert np.all(np.abs(mine.astype(np.float64) - ref) <= 2.5e-7 + t * 1.5e-7)
    assert np.array_equal(mine[0], ref[0])                      # t = 0: exactly (1, 0, 1, 0, ...)


def test_rope_header_rejects_shapes_a_vector_would_straddle():
    with pytest.raises(ValueError):
        headers.rope_header(16, 4, 4, 6, "fp32")                # head_dim/2 = 3 pairs, vectors hold 2
    with pytest.raises(ValueError):
        headers.rope_header(16, 4, 4, 12, "bf16")               # 6 pairs, vectors hold 4
    with pytest.raises(ValueError):
        headers.rope_header(16, 4, 4, 12, "fp16")               # likewise
    with pytest.raises(ValueError):
        headers.rope_header(16, 4, 4, 64, "fp8")                # no such storage type
    with pytest.raises(ValueError):
        headers.rope_header(16, 4, 4, 64, "fp32", layout="nope")
    text = headers.rope_header(1024, 12, 12, 64, "fp32", "qkv").decode()
    assert "rope_heads = 36" in text and "rope_rotated = 24" in text and "rope_half = 32" in text
    text = headers.rope_header(4096, 32, 0, 128, "bf16", "heads", backward=True).decode()
    assert "x_re * c + x_im * s" in text and "x_im * c - x_re * s" in text   # conjugate rotation
