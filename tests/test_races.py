"""Data races in the host code, hunted on the CPU with ThreadSanitizer.

Two drivers: the allocator's policy code over the fake backing store with six threads allocating,
freeing, trimming and reading statistics on one pool; and the library's own translation units
(registry, tuning knobs, configuration setters, error slot, run-time compiler) with six threads
registering headers, changing knobs and compiling at once through the C ABI.  The second driver
also runs under AddressSanitizer and UBSan.  No GPU is involved: neither driver makes a device
call that needs one.
"""
import os
import shutil
import subprocess

import pytest

from l2_torch_alloc_amd import build as sa_build

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
NATIVE = os.path.join(HERE, "native")
CSRC = os.path.join(ROOT, "l2_torch_alloc_amd", "csrc")
ENV = dict(os.environ, TSAN_OPTIONS="halt_on_error=1 exitcode=66 second_deadlock_stack=1",
           SIDEAWARE_NO_DISK_CACHE="1")


def run(exe):
    proc = subprocess.run([exe], capture_output=True, text=True, timeout=900, env=ENV)
    assert "ThreadSanitizer" not in proc.stderr, proc.stderr[-6000:]
    assert proc.returncode == 0, (proc.returncode, proc.stdout[-2000:], proc.stderr[-4000:])
    return proc.stdout


def test_pool_under_thread_sanitizer(tmp_path):
    exe = str(tmp_path / "pool_tsan")
    subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=thread", "-pthread",
                    os.path.join(NATIVE, "pool_tsan_main.cpp"), os.path.join(CSRC, "pool.cpp"), "-o", exe],
                   check=True, capture_output=True, text=True)
    out = run(exe)
    assert "bad=0 live=0 backing_used=0" in out


def test_registry_tuning_and_compiler_under_thread_sanitizer(tmp_path):
    hipcc = shutil.which("hipcc") or os.path.join(sa_build.rocm_root(), "bin", "hipcc")
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not found")
    sa_build.generate_template_literal()
    exe = str(tmp_path / "registry_tsan")
    lib_dir = os.path.join(sa_build.rocm_root(), "lib")
    cmd = [hipcc, "--offload-arch=gfx950", "-std=c++17", "-O1", "-g", "-Xarch_host", "-fsanitize=thread",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-pthread",
           os.path.join(NATIVE, "registry_tsan_main.cpp")] + \
          [os.path.join(CSRC, s) for s in sa_build.SOURCES] + \
          ["-L" + lib_dir, "-lhiprtc", "-Wl,-rpath," + lib_dir, "-o", exe]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-4000:]
    out = run(exe)
    assert "bad=0" in out


def test_registry_and_compiler_under_address_and_undefined_behaviour_sanitizers(tmp_path):
    # the same driver, host code only, for memory errors instead of races: the registry, the ELF
    # symbol reader of the run-time compiler, the configuration text, the error slot
    hipcc = shutil.which("hipcc") or os.path.join(sa_build.rocm_root(), "bin", "hipcc")
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not found")
    sa_build.generate_template_literal()
    exe = str(tmp_path / "registry_asan")
    lib_dir = os.path.join(sa_build.rocm_root(), "lib")
    cmd = [hipcc, "--offload-arch=gfx950", "-std=c++17", "-O1", "-g",
           "-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined",
           "-Xarch_host", "-fno-sanitize-recover=undefined",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-pthread",
           os.path.join(NATIVE, "registry_tsan_main.cpp")] + \
          [os.path.join(CSRC, s) for s in sa_build.SOURCES] + \
          ["-L" + lib_dir, "-lhiprtc", "-Wl,-rpath," + lib_dir, "-o", exe]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-4000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0", UBSAN_OPTIONS="print_stacktrace=1",
               SIDEAWARE_NO_DISK_CACHE="1")
    run_ = subprocess.run([exe], capture_output=True, text=True, timeout=900, env=env)
    assert "AddressSanitizer" not in run_.stderr and "runtime error" not in run_.stderr, run_.stderr[-6000:]
    assert run_.returncode == 0 and "bad=0" in run_.stdout, (run_.returncode, run_.stdout[-2000:], run_.stderr[-4000:])


def test_pool_under_address_and_undefined_behaviour_sanitizers(tmp_path):
    # the allocator's policy code with the same six-thread driver, for memory errors
    exe = str(tmp_path / "pool_asan")
    subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
                    "-pthread", os.path.join(NATIVE, "pool_tsan_main.cpp"), os.path.join(CSRC, "pool.cpp"), "-o", exe],
                   check=True, capture_output=True, text=True)
    proc = subprocess.run([exe], capture_output=True, text=True, timeout=900,
                          env=dict(os.environ, UBSAN_OPTIONS="print_stacktrace=1"))
    assert "AddressSanitizer" not in proc.stderr and "runtime error" not in proc.stderr, proc.stderr[-6000:]
    assert proc.returncode == 0 and "bad=0 live=0 backing_used=0" in proc.stdout, (proc.returncode, proc.stdout[-2000:])
