"""The source-level adapter (llumnix-kv_amd/adapter/kvt_blade_adapter.hpp) hands
out functions with the reference's ParseBlockFunc signature. Here they are
called side by side with the reference's own functions on the very same
WorkerInfo / ReqSendTask objects (oracle/adapter_check.cpp, built by
`make -C oracle adapter` where the reference checkout exists): same ranges,
same exception class. CPU only; skipped where the checker was never built."""
import ctypes as C
import json
import os

import pytest

import cases
import checkers
import kvt_amd
from kvt_amd.ctypes_defs import Task, WorkerInfo, task_array

SO = os.path.join(checkers.ROOT, "oracle", "_ref", "libkvt_adapter_check.so")
pytestmark = pytest.mark.skipif(not os.path.exists(SO), reason="adapter checker not built")

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "parse_golden.json")


def _lib():
    kvt_amd.lib()                      # maps the product library (and one HIP runtime) first
    lib = C.CDLL(SO)
    lib.kvtadp_compare.argtypes = [C.c_int, C.POINTER(WorkerInfo), C.POINTER(WorkerInfo),
                                   C.c_uint32, C.c_uint32, C.c_uint32, C.POINTER(Task),
                                   C.c_uint32, C.POINTER(C.c_int), C.POINTER(C.c_uint64)]
    lib.kvtadp_compare.restype = C.c_int
    return lib


def _compare(lib, case):
    pid, src, dst, valid, tps, tpr, tasks = cases.materialise(case)
    arr = task_array(tasks)
    ref_rc, n = C.c_int(), C.c_uint64()
    rc = lib.kvtadp_compare(pid, C.byref(src), C.byref(dst), valid, tps, tpr, arr, len(tasks),
                            C.byref(ref_rc), C.byref(n))
    return rc, ref_rc.value, n.value


@pytest.mark.parametrize("parser", cases.ALL_PARSERS)
def test_adapter_equals_reference_function(parser):
    lib = _lib()
    ranges = errors = 0
    for seed in range(3000, 3150):
        case = cases.gen_case(parser, seed)
        if case["fp8"]:
            continue                   # the reference latches the conversion switch from the environment
        rc, ref_rc, n = _compare(lib, case)
        assert rc == 0, (case["name"], rc, ref_rc)
        ranges += n
        errors += ref_rc != 0
    assert ranges > 0


def test_adapter_on_the_golden_cases():
    lib = _lib()
    with open(GOLDEN) as f:
        golden = json.load(f)
    for case in golden:
        if case["fp8"]:
            continue
        rc, ref_rc, n = _compare(lib, case)
        assert rc == 0, case["name"]
        assert (ref_rc != 0) == (case["rc"] != 0)


def test_adapter_hands_the_memcpy_variables_to_the_library(monkeypatch):
    """BLLM_KVTRANS_COPY_MEMCPY_BLOCK_THRESHOLD_BYTES / _MAX_BLOCKS (copy_kernels.cpp:496-499):
    set values replace the library's thresholds, unset or unparsable ones leave them alone."""
    lib, k = _lib(), kvt_amd.lib()
    a, b = C.c_uint64(), C.c_uint64()

    def current():
        assert k.kvt_get_copy_memcpy_thresholds(C.byref(a), C.byref(b)) == 0
        return a.value, b.value

    try:
        monkeypatch.delenv("BLLM_KVTRANS_COPY_MEMCPY_BLOCK_THRESHOLD_BYTES", raising=False)
        monkeypatch.delenv("BLLM_KVTRANS_COPY_MEMCPY_MAX_BLOCKS", raising=False)
        assert lib.kvtadp_apply_copy_memcpy_env() == 0 and current() == (8 << 20, 16)
        monkeypatch.setenv("BLLM_KVTRANS_COPY_MEMCPY_BLOCK_THRESHOLD_BYTES", "262144")
        assert lib.kvtadp_apply_copy_memcpy_env() == 0 and current() == (262144, 16)
        monkeypatch.setenv("BLLM_KVTRANS_COPY_MEMCPY_MAX_BLOCKS", "4")
        monkeypatch.setenv("BLLM_KVTRANS_COPY_MEMCPY_BLOCK_THRESHOLD_BYTES", "12k")   # not a number
        assert lib.kvtadp_apply_copy_memcpy_env() == 0 and current() == (262144, 4)
        monkeypatch.setenv("BLLM_KVTRANS_COPY_MEMCPY_MAX_BLOCKS", "0")               # route off
        assert lib.kvtadp_apply_copy_memcpy_env() == 0 and current() == (262144, 0)
    finally:
        assert k.kvt_reset_copy_memcpy_thresholds() == 0
