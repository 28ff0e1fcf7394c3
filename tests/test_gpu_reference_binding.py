"""The library bound exactly as the reference's own script binds its `sideaware.so` (test.py:14-39):
opened as `./sideaware.so` from the working directory, through PyTorch's pluggable allocator and
through ctypes, `sideband_value` declared pointer-sized, and the `torch.cuda.Stream` object itself
passed as the stream.  The host program is tests/native/reference_style_host.py; it needs a process
of its own because the allocator can only be installed before a process's first device allocation."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)


def test_a_script_written_for_the_reference_runs_against_this_library(tmp_path):
    lib = os.path.join(ROOT, "l2_torch_alloc_amd", "sideaware.so")
    assert os.path.exists(lib), "sideaware.so is not built"
    os.symlink(lib, tmp_path / "sideaware.so")
    print("reference-style host in", tmp_path, flush=True)
    proc = subprocess.run([sys.executable, os.path.join(HERE, "native", "reference_style_host.py")],
                          cwd=tmp_path, capture_output=True, text=True, timeout=170)
    assert proc.returncode == 0, proc.stdout[-3000:] + proc.stderr[-3000:]
    lines = proc.stdout.splitlines()
    assert lines[-1] == "done" and not any(l.startswith("FAILED") for l in lines)
    assert sum(l.startswith("ok: ") for l in lines) == 10, proc.stdout
