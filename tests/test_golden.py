"""The committed golden vectors are reproducible from the CPU oracle, bit for bit."""
import importlib.util
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden")

spec = importlib.util.spec_from_file_location("make_golden", os.path.join(GOLDEN, "make_golden.py"))
make_golden = importlib.util.module_from_spec(spec)
spec.loader.exec_module(make_golden)


@pytest.mark.parametrize("name", sorted(make_golden.CASES))
def test_rope_fixture_reproduces(name):
    stored = np.load(os.path.join(GOLDEN, name + ".npz"))
    fresh = make_golden.make(name)
    assert sorted(stored.files) == sorted(fresh)
    for key in stored.files:
        a, b = stored[key], np.asarray(fresh[key])
        assert a.dtype == b.dtype and a.shape == b.shape, key
        assert a.tobytes() == b.tobytes(), key


def test_scale_bias_fixture_reproduces():
    stored = np.load(os.path.join(GOLDEN, "scale_bias_bf16.npz"))
    fresh = make_golden.scale_bias_case()
    for key in stored.files:
        assert stored[key].tobytes() == np.asarray(fresh[key]).tobytes(), key
