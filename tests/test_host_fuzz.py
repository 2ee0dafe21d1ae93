"""Builds tests/host_fuzz.cpp with AddressSanitizer + UndefinedBehaviorSanitizer
together with the product's host-side sources (no HIP needed) and runs it: the C
ABI must survive malformed frames, garbage geometries and bad block tables
without a memory error, and its invariants must hold. tests/plan_fuzz.cpp does
the same for the copy-plan builder, which lives in HIP translation units: hipcc
builds them with the sanitizers on the host side only, and host-only plans
(device = -1) need no GPU. tests/thread_check.cpp runs the host entry points
from eight threads that share parsers, under ThreadSanitizer. CPU only."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "llumnix-kv_amd", "csrc")
HOST_SOURCES = ["kvt_parse.cpp", "kvt_parse_build.cpp", "kvt_ranges.cpp", "kvt_wire.cpp", "kvt_runs.cpp"]


def test_host_entry_points_under_sanitizers(tmp_path):
    exe = str(tmp_path / "host_fuzz")
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fno-omit-frame-pointer",
           "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
           "-I", os.path.join(ROOT, "include"), "-I", CSRC,
           os.path.join(ROOT, "tests", "host_fuzz.cpp")]
    cmd += [os.path.join(CSRC, s) for s in HOST_SOURCES] + ["-o", exe]
    subprocess.check_call(cmd)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=1",
               UBSAN_OPTIONS="print_stacktrace=1")
    for seed in ("12345", "777"):
        res = subprocess.run([exe, "2", seed], capture_output=True, text=True, env=env, timeout=600)
        assert res.returncode == 0, res.stdout[-2000:] + res.stderr[-6000:]
        assert "host fuzz ok" in res.stdout


def test_shared_parsers_under_thread_sanitizer(tmp_path):
    exe = str(tmp_path / "thread_check")
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=thread",
           "-I", os.path.join(ROOT, "include"), "-I", CSRC,
           os.path.join(ROOT, "tests", "thread_check.cpp")]
    cmd += [os.path.join(CSRC, s) for s in HOST_SOURCES] + ["-o", exe, "-lpthread"]
    subprocess.check_call(cmd)
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=1:abort_on_error=1")
    res = subprocess.run([exe, "40", "31337"], capture_output=True, text=True, env=env, timeout=600)
    assert res.returncode == 0, res.stdout[-2000:] + res.stderr[-6000:]
    assert "thread check ok" in res.stdout


HIPCC = shutil.which("hipcc") or ("/opt/rocm/bin/hipcc" if os.path.exists("/opt/rocm/bin/hipcc") else None)


@pytest.mark.skipif(HIPCC is None, reason="hipcc not installed")
def test_plan_builder_under_sanitizers(tmp_path):
    exe = str(tmp_path / "plan_fuzz")
    cmd = [HIPCC, "--offload-arch=gfx950", "-O1", "-g", "-std=c++17",
           "-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined",
           "-Xarch_host", "-fno-sanitize-recover=all",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-I", os.path.join(ROOT, "include"), "-I", CSRC,
           os.path.join(ROOT, "tests", "plan_fuzz.cpp")]
    cmd += [os.path.join(CSRC, s) for s in ["kvt_plan.hip", "kvt_runtime.hip", "kvt_kernels.hip", "kvt_object_ring.hip", "kvt_dropin.hip"] + HOST_SOURCES]
    cmd += ["-o", exe]
    subprocess.run(cmd, check=True, capture_output=True)
    # (no leak check: the HIP runtime keeps its own allocations for the life of the process)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=1",
               UBSAN_OPTIONS="print_stacktrace=1")
    for seed in ("2024", "99"):
        res = subprocess.run([exe, "1", seed], capture_output=True, text=True, env=env, timeout=600)
        assert res.returncode == 0, res.stdout[-2000:] + res.stderr[-6000:]
        assert "plan fuzz ok" in res.stdout
