"""Builds ``sideaware.so`` for gfx950 with hipcc (no GPU needed: hipcc cross-compiles).

``python -m l2_torch_alloc_amd.build`` or ``build_library()``.  The only generated file is the
kernel template wrapped in a C++ raw string literal so the library can hand it to hipRTC.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "sideaware.so")

SOURCES = ["sideaware.hip", "side_map.hip", "pool.cpp", "hip_backing.cpp", "rtc.cpp"]
DEPENDS = SOURCES + ["pool.h", "hip_backing.h", "rtc.h", "side_map.h", "launch_plan.h", "elementwise_kernel.hip.inc",
                     os.path.join("..", "..", "include", "sideaware.h")]


def rocm_root() -> str:
    return os.environ.get("ROCM_PATH") or "/opt/rocm"


def _hipcc() -> str:
    exe = shutil.which("hipcc") or os.path.join(rocm_root(), "bin", "hipcc")
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; sideaware.so can only be built with ROCm installed")
    return exe


def generate_template_literal() -> str:
    """Wraps the kernel template in a raw string literal for inclusion by sideaware.hip."""
    src = os.path.join(CSRC, "elementwise_kernel.hip.inc")
    dst = os.path.join(CSRC, "elementwise_kernel.generated.inc")
    with open(src) as f:
        text = f.read()
    assert ')SA_KERNEL"' not in text
    body = 'R"SA_KERNEL(' + text + ')SA_KERNEL"\n'
    if not os.path.exists(dst) or open(dst).read() != body:
        with open(dst, "w") as f:
            f.write(body)
    return dst


def needs_build() -> bool:
    if not os.path.exists(LIB_PATH):
        return True
    built = os.path.getmtime(LIB_PATH)
    return any(os.path.getmtime(os.path.join(CSRC, d)) > built for d in DEPENDS)


def build_library(force: bool = True, verbose: bool = False) -> str:
    """Compiles the library in-tree and returns its path."""
    if not force and not needs_build():
        return LIB_PATH
    generate_template_literal()
    cmd = [
        _hipcc(), "--offload-arch=gfx950", "-std=c++17", "-O2", "-fPIC", "-shared",
        # keep the compiler from forming packed fp32 instructions out of scalar code
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        "-Wall", "-Wno-unused-result",
        "-fvisibility=hidden",
    ]
    cmd += [os.path.join(CSRC, s) for s in SOURCES]
    cmd += ["-L" + os.path.join(rocm_root(), "lib"), "-lhiprtc",
            "-Wl,-rpath," + os.path.join(rocm_root(), "lib"),
            "-o", LIB_PATH + ".tmp"]
    if verbose:
        print(" ".join(cmd), file=sys.stderr)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "packed-fp32-ops' is not a recognized feature"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + err)
    if verbose and err.strip():
        print(err, file=sys.stderr)
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(force=True, verbose=True))
