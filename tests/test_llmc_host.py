"""A compiled C++ host in the shape of the reference's llm.c benchmark (example_llmc_rope.cu:132-144,
:243-316) against the shared library: sideaware_malloc, a one-line `#include "file"` op header
resolved in the working directory, an in-place sideaware_elementwise launch, forward and backward
held against the CPU oracle (llm.c's tolerance rule, and bit for bit).  The link step runs
anywhere; running the program needs the GPU.
"""
import os
import subprocess

import pytest

from l2_torch_alloc_amd import build as sa_build
from l2_torch_alloc_amd import headers
from oracle import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")


def build_host(tmp_path):
    lib_dir = os.path.dirname(sa_build.build_library(force=False))
    oracle_dir = os.path.dirname(oracle.build())
    exe = tmp_path / "llmc_rope_host"
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-D__HIP_PLATFORM_AMD__", "-I" + ROCM + "/include",
                    os.path.join(ROOT, "tests", "native", "llmc_rope_host.cpp"),
                    "-L" + lib_dir, "-l:sideaware.so", "-L" + oracle_dir, "-l:liboracle.so",
                    "-L" + ROCM + "/lib", "-lamdhip64",
                    "-Wl,-rpath," + lib_dir + ":" + oracle_dir + ":" + ROCM + "/lib", "-o", str(exe)], check=True)
    return exe


def test_llmc_style_host_compiles_and_links(tmp_path):
    exe = build_host(tmp_path)
    proc = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert proc.returncode == 2 and "usage" in proc.stderr        # no arguments: prints usage, touches no device


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(8, 1024, 32, 128), (2, 96, 6, 64)])
def test_llmc_style_host_matches_the_oracle(tmp_path, shape):
    B, T, NH, HS = shape
    exe = build_host(tmp_path)
    (tmp_path / "rope_fwd.h").write_bytes(headers.rope_header(T, NH, NH, HS, "fp32", "qkv"))
    (tmp_path / "rope_bwd.h").write_bytes(headers.rope_header(T, NH, NH, HS, "fp32", "qkv", backward=True))
    print("llmc host, shape", shape, flush=True)
    proc = subprocess.run([str(exe), "rope_fwd.h", "rope_bwd.h", str(B), str(T), str(NH), str(HS)],
                          cwd=tmp_path, capture_output=True, text=True, timeout=110)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "llmc rope host ok" in proc.stdout
    assert proc.stdout.count("0 faults, 0 values differ") == 3
    isa = (tmp_path / "isa.txt").read_text()                       # sideaware_write_sass took effect
    assert "sideaware_rope_fwd_fp32_qkv" in isa and "global_load_dwordx4" in isa
