"""Builds tests/host_fuzz.cpp with AddressSanitizer + UndefinedBehaviorSanitizer
together with the product's host-side sources (no HIP needed) and runs it: the C
ABI must survive malformed frames, garbage geometries and bad block tables
without a memory error, and its invariants must hold. CPU only."""
import os
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
