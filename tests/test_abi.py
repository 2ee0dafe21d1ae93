"""CPU-side checks of the C ABI: the library loads without a GPU, exports every
symbol include/kvt_hip.h declares, struct sizes agree with the ctypes mirrors,
and device entry points fail loudly (never fall back) when no gfx950 is present."""
import ctypes as C
import os
import re

import pytest

import kvt_amd
from kvt_amd import binding
from kvt_amd.ctypes_defs import IpcBlock, ParseOpts, Task, WorkerInfo, make_worker_info

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "kvt_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(kvt_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_what_the_binding_binds():
    assert _declared_symbols() == sorted(binding.SIGNATURES)


def test_library_exports_every_declared_symbol():
    lib = kvt_amd.lib()
    for name in _declared_symbols():
        assert hasattr(lib, name), name


def test_struct_sizes_match():
    lib = kvt_amd.lib()
    assert lib.kvt_abi_sizeof(0) == C.sizeof(IpcBlock) == 24
    assert lib.kvt_abi_sizeof(1) == C.sizeof(WorkerInfo)
    assert lib.kvt_abi_sizeof(2) == C.sizeof(Task)
    assert lib.kvt_abi_sizeof(3) == C.sizeof(ParseOpts)
    assert lib.kvt_abi_sizeof(4) == C.sizeof(binding.Xform)


def test_null_arguments_are_errors_not_crashes():
    lib = kvt_amd.lib()
    assert lib.kvt_parse_block(None, None, None) == 3
    assert lib.kvt_block_lists_view(None, 0, None, None) == 3
    assert b"null" in lib.kvt_last_error()
    lists = kvt_amd.BlockLists()
    data, n = C.POINTER(IpcBlock)(), C.c_uint64()
    assert lib.kvt_block_lists_view(lists.h, 0, C.byref(data), C.byref(n)) == 1


def test_unknown_parser_id_is_refused():
    w = make_worker_info([16384], [1024], 8)
    for pid in (-1, 25, 1000):
        with pytest.raises(kvt_amd.KvtError) as e:
            kvt_amd.Parser(pid, w, w, 1, 1, 0)
        assert e.value.code == 4


@pytest.mark.skipif(kvt_amd.device_count() > 0, reason="this check is for machines without a GPU")
def test_gpu_entry_points_fail_loudly_without_a_device():
    w = make_worker_info([65536], [4096], 8)
    lists = kvt_amd.BlockLists()
    p = kvt_amd.Parser(4, w, w, 1, 1, 0)
    from kvt_amd.ctypes_defs import TaskBuf
    assert p.parse(TaskBuf(0, 16, True, [[1]], [[2]]).struct, lists) == 0
    with pytest.raises(kvt_amd.KvtError) as e:
        kvt_amd.Plan(0, lists, [65536 * 8], [65536 * 8])
    assert e.value.code == 6
    with pytest.raises(kvt_amd.KvtError) as e:
        kvt_amd.Stager(0, 4096, 2)
    assert e.value.code == 6
    assert kvt_amd.lib().kvt_copy_linear(1, 1, 16, None) == 6
    assert kvt_amd.lib().kvt_set_copy_cu_usage(0, 0.5) == 6


def test_memcpy_route_thresholds_are_process_wide_settings():
    import ctypes as C
    lib = kvt_amd.lib()
    a, b = C.c_uint64(), C.c_uint64()
    assert lib.kvt_get_copy_memcpy_thresholds(C.byref(a), C.byref(b)) == 0
    assert (a.value, b.value) == (8 << 20, 16)
    try:
        assert lib.kvt_set_copy_memcpy_thresholds(256 << 10, 4) == 0
        assert lib.kvt_get_copy_memcpy_thresholds(C.byref(a), None) == 0 and a.value == 256 << 10
        assert lib.kvt_get_copy_memcpy_thresholds(None, C.byref(b)) == 0 and b.value == 4
        assert lib.kvt_set_copy_memcpy_thresholds(0, 4) != 0          # every range would qualify
        assert lib.kvt_get_copy_memcpy_thresholds(C.byref(a), C.byref(b)) == 0
        assert (a.value, b.value) == (256 << 10, 4)
        assert lib.kvt_set_copy_memcpy_thresholds(1, 0) == 0          # route switched off
    finally:
        assert lib.kvt_reset_copy_memcpy_thresholds() == 0


def test_launcher_stand_in_exports_the_reference_names():
    """libkvt_blade_launchers.so: the extern "C" names kvtransfer/src/copy_kernels.cpp:52-85,
    101-108 declares (no calls here: they launch kernels)."""
    import ctypes as C
    import os
    kvt_amd.lib()
    shim = C.CDLL(os.path.join(os.path.dirname(kvt_amd.LIB_PATH), "libkvt_blade_launchers.so"))
    for name in ("launch_copy_int64_array_h2d_kernel", "launch_copy_h2d_direct_kernel",
                 "launch_copy_d2h_direct_kernel", "launch_copy_d2h_bf16_to_fp8_kernel"):
        assert hasattr(shim, name), name


def test_cached_load_threshold_is_a_process_wide_setting():
    lib = kvt_amd.lib()
    assert lib.kvt_get_copy_cached_load_max() == 0
    try:
        assert lib.kvt_set_copy_cached_load_max(0) == 0 and lib.kvt_get_copy_cached_load_max() == 0
        assert lib.kvt_set_copy_cached_load_max(1 << 40) == 0
        assert lib.kvt_get_copy_cached_load_max() == 1 << 40
    finally:
        assert lib.kvt_set_copy_cached_load_max(0) == 0
