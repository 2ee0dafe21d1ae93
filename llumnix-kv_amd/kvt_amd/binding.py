"""ctypes declarations for every symbol of include/kvt_hip.h plus small RAII wrappers."""
import ctypes as C
import importlib.util
import os
import sys

import numpy as np

from .ctypes_defs import IpcBlock, ParseOpts, Task, WorkerInfo

LIB_PATH = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "libkvt_hip.so")

_vp = C.c_void_p
_u32, _u64, _i64, _int = C.c_uint32, C.c_uint64, C.c_int64, C.c_int
_P = C.POINTER


class WireLayout(C.Structure):
    _fields_ = [("total_bytes", _u64), ("n_tensors", _u32), ("reserved0", _u32),
                ("meta_offset", _u64 * 8), ("blob_offset", _u64 * 8), ("blob_bytes", _u64 * 8)]


WIRE_TCP, WIRE_RDMA_STAGED = 0, 1


class SlotLayout(C.Structure):
    _fields_ = [("n_entries", _u64), ("layer_bytes", _u64), ("n_tensors", _u32), ("reserved0", _u32),
                ("tensor_bytes", _u64 * 8), ("tensor_offset", _u64 * 8)]


class Xform(C.Structure):
    _fields_ = [("kind", _u32), ("heads", _u32), ("ntpb", _u32), ("row_bytes", _u32)]


# name -> (restype, argtypes); this table is also what tests/test_abi.py checks
# against the declarations in include/kvt_hip.h.
SIGNATURES = {
    "kvt_last_error": (C.c_char_p, []),
    "kvt_abi_sizeof": (_u64, [_int]),
    "kvt_device_count": (_int, []),
    "kvt_compute_valid_ranks_pd": (_u32, [_u32, _u32, C.c_int32]),
    "kvt_select_parser": (_int, [_int, _P(WorkerInfo), _P(WorkerInfo), _P(_u32), _P(_u32),
                                 _P(_u32), _P(_int), _P(_int)]),
    "kvt_parser_create": (_int, [_int, _P(WorkerInfo), _P(WorkerInfo), _u32, _u32, _u32,
                                 _P(ParseOpts), _P(_vp)]),
    "kvt_parser_destroy": (None, [_vp]),
    "kvt_block_lists_create": (_int, [_P(_vp)]),
    "kvt_block_lists_destroy": (None, [_vp]),
    "kvt_block_lists_clear": (None, [_vp]),
    "kvt_block_lists_num_tensors": (_u32, [_vp]),
    "kvt_block_lists_view": (_int, [_vp, _u32, _P(_P(IpcBlock)), _P(_u64)]),
    "kvt_block_lists_append": (_int, [_vp, _u32, _vp, _u64]),
    "kvt_parse_block": (_int, [_vp, _P(Task), _vp]),
    "kvt_merge_interval": (_int, [_vp, _u64, _P(_u64), _P(_u64)]),
    "kvt_block_lists_merge": (_int, [_vp]),
    "kvt_validate_ipc_block_bounds": (_int, [_vp, _u64, _u64, _int, _u64, _P(_u64)]),
    "kvt_cache_register": (_int, [_int, _P(_vp), _u32, _u32, _P(_u64), _P(_vp)]),
    "kvt_cache_destroy": (None, [_vp]),
    "kvt_plan_create": (_int, [_int, _vp, _P(_u64), _P(_u64), _P(Xform), _u32, _P(_vp)]),
    "kvt_plan_destroy": (None, [_vp]),
    "kvt_plan_ready": (_int, [_vp]),
    "kvt_plan_num_tensors": (_u32, [_vp]),
    "kvt_plan_num_chunks": (_u64, [_vp]),
    "kvt_plan_tensor_bytes": (_u64, [_vp, _u32]),
    "kvt_plan_tensor_offset": (_u64, [_vp, _u32]),
    "kvt_plan_layer_bytes": (_u64, [_vp]),
    "kvt_pack": (_int, [_vp, _vp, _u32, _u32, _vp, _u64, _vp]),
    "kvt_unpack": (_int, [_vp, _vp, _u32, _u32, _vp, _u64, _vp]),
    "kvt_run_lists_create": (_int, [_P(_vp)]),
    "kvt_run_lists_destroy": (None, [_vp]),
    "kvt_run_lists_clear": (None, [_vp]),
    "kvt_run_lists_num_tensors": (_u32, [_vp]),
    "kvt_run_lists_view": (_int, [_vp, _u32, _P(_vp), _P(_u64)]),
    "kvt_run_lists_append": (_int, [_vp, _u32, _vp, _u64]),
    "kvt_run_lists_totals": (_int, [_vp, _u32, _P(_u64), _P(_u64)]),
    "kvt_parse_block_runs": (_int, [_vp, _P(Task), _vp]),
    "kvt_run_lists_expand": (_int, [_vp, _vp]),
    "kvt_run_lists_compress": (_int, [_vp, _vp]),
    "kvt_plan_create_runs": (_int, [_int, _vp, _P(_u64), _P(_u64), _u32, _P(_vp)]),
    "kvt_plan_create_runs_bf16_to_fp8": (_int, [_int, _vp, _P(_u64), _P(_u64), _u32, _P(_vp)]),
    "kvt_plan_num_strided_chunks": (_u64, [_vp]),
    "kvt_plan_create_objects": (_int, [_int, _vp, _P(_u64), _P(_u64), _u64, _u64, _u32, _P(_vp)]),
    "kvt_plan_host_tables": (_int, [_vp, _P(_vp), _P(_u64), _P(_u32), _P(_vp)]),
    "kvt_plan_slot_create": (_int, [_int, _u32, _P(_u64), _P(_u64), _P(Xform), _u32, _u64, _u64,
                                    _P(_vp)]),
    "kvt_plan_slot_create_runs": (_int, [_int, _u32, _P(_u64), _P(_u64), _u32, _int, _u64, _u64,
                                         _P(_vp)]),
    "kvt_plan_slot_fill": (_int, [_vp, _vp, _vp, _P(SlotLayout)]),
    "kvt_plan_slot_fill_runs": (_int, [_vp, _vp, _vp, _P(SlotLayout)]),
    "kvt_get_copy_ticket_stats": (_int, [_int, _P(_u64)]),
    "kvt_pack_at": (_int, [_vp, _vp, _u32, _u32, _vp, _u64, _P(_u64), _vp]),
    "kvt_unpack_at": (_int, [_vp, _vp, _u32, _u32, _vp, _u64, _P(_u64), _vp]),
    "kvt_wire_layout_of": (_int, [_int, _vp, _P(WireLayout)]),
    "kvt_wire_write_frame": (_int, [_int, _vp, _u64, _u64, _u64, _vp, _P(WireLayout)]),
    "kvt_wire_parse_frame": (_int, [_int, _vp, _u64, _u32, _P(_u64), _P(_u64), _vp,
                                    _P(WireLayout)]),
    "kvt_block_object_lists": (_int, [_int, _P(WorkerInfo), _P(WorkerInfo), _vp, _vp, _u64, _vp,
                                      _P(_u64)]),
    "kvt_enlarge_block_ids": (_int, [_vp, _u64, _u32, _vp]),
    "kvt_launch_copy_d2h_direct": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _int, _int, _vp]),
    "kvt_launch_copy_h2d_direct": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _int, _int, _vp]),
    "kvt_launch_copy_d2h_bf16_to_fp8": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _int, _int, _vp]),
    "kvt_launch_copy_int64_array_h2d": (_int, [_vp, _vp, _i64, _int, _int, _vp]),
    "kvt_initialize_copy_method_profile": (_int, [_int]),
    "kvt_object_ring_create": (_int, [_int, _u64, _u32, _u32, _P(_vp)]),
    "kvt_object_ring_destroy": (None, [_vp]),
    "kvt_object_ring_entry": (_vp, [_vp, _u32]),
    "kvt_object_ring_reserve": (_int, [_vp, _vp, _u32, _vp, _vp]),
    "kvt_object_ring_save": (_int, [_vp, _vp, _u32, _vp, _u64, _vp]),
    "kvt_object_ring_commit": (_int, [_vp, _vp, _u32]),
    "kvt_object_ring_lookup": (_int, [_vp, _vp, _u32, _vp, _vp]),
    "kvt_object_ring_load": (_int, [_vp, _vp, _vp, _u32, _vp, _u64, _vp]),
    "kvt_object_ring_release": (_int, [_vp, _vp, _u32]),
    "kvt_object_ring_wait": (_int, [_vp, _u32]),
    "kvt_object_ring_stats": (_int, [_vp, _vp]),
    "kvt_set_copy_memcpy_thresholds": (_int, [_u64, _u64]),
    "kvt_get_copy_memcpy_thresholds": (_int, [_P(_u64), _P(_u64)]),
    "kvt_reset_copy_memcpy_thresholds": (_int, []),
    "kvt_get_copy_method_profile": (_int, [_int] + [_P(C.c_double)] * 4 + [_P(_u64), _P(_int), _P(C.c_double)]),
    "kvt_set_copy_cached_load_max": (_int, [_u64]),
    "kvt_get_copy_cached_load_max": (_u64, []),
    "kvt_set_copy_cached_store_max": (_int, [_u64]),
    "kvt_get_copy_cached_store_max": (_u64, []),
    "kvt_set_copy_cu_usage": (_int, [_int, C.c_double]),
    "kvt_get_copy_cu_usage": (_int, [_int, _P(C.c_double), _P(_u32)]),
    "kvt_get_kernel_copy_buffer": (_int, [_int, _i64, _P(_vp), _P(_vp)]),
    "kvt_get_thread_local_stream": (_int, [_int, _int, _P(_vp)]),
    "kvt_copy_handle_data_with_kernel": (_int, [_vp, _vp, _vp, _u64, _u64, _int, _int, _vp, _vp,
                                               _vp, _i64]),
    "kvt_copy_handle_data_kernel_direct": (_int, [_vp, _vp, _vp, _u64, _u64, _int, _int, _vp, _vp,
                                                  _vp, _vp, _vp, _int]),
    "kvt_copy_handle_data_kernel_direct_static": (_int, [_vp, _vp, _vp, _u64, _u64, _int, _int, _vp,
                                                         _vp, _int]),
    "kvt_copy_d2h_bf16_to_fp8": (_int, [_vp, _vp, _vp, _u64, _u64, _int, _vp, _vp, _vp, _i64]),
    "kvt_session_create": (_int, [_vp, _vp, _vp, _u64, _P(_vp)]),
    "kvt_session_destroy": (None, [_vp]),
    "kvt_session_save_layer": (_int, [_vp, _u32, _vp]),
    "kvt_session_save_layer_event": (_int, [_vp, _u32, _vp]),
    "kvt_session_save_layers": (_int, [_vp, _u32, _u32, _vp]),
    "kvt_session_save_layers_inline": (_int, [_vp, _u32, _u32, _vp]),
    "kvt_session_wait_layer": (_int, [_vp, _u32]),
    "kvt_session_wait_layer_step": (_int, [_vp, _u64, _u32]),
    "kvt_session_wait_layer_for": (_int, [_vp, _u64, _u32, _u64]),
    "kvt_session_begin_step": (_int, [_vp, _P(_u64)]),
    "kvt_session_set_plan": (_int, [_vp, _vp, _vp, _u64]),
    "kvt_session_join": (_int, [_vp, _vp]),
    "kvt_session_side_stream": (_vp, [_vp]),
    "kvt_stager_create": (_int, [_int, _u64, _u32, _P(_vp)]),
    "kvt_stager_destroy": (None, [_vp]),
    "kvt_stager_slot": (_vp, [_vp, _u32]),
    "kvt_stager_copy_stream": (_vp, [_vp]),
    "kvt_stager_save": (_int, [_vp, _u32, _vp, _u64, _vp]),
    "kvt_stager_save_at": (_int, [_vp, _u32, _u64, _vp, _u64, _vp]),
    "kvt_stager_load_at": (_int, [_vp, _u32, _u64, _vp, _u64, _vp]),
    "kvt_stager_load": (_int, [_vp, _u32, _vp, _u64, _vp]),
    "kvt_stager_wait": (_int, [_vp, _u32]),
    "kvt_measure_pcie": (_int, [_int, _int, _u64, _u32, _P(C.c_double)]),
    "kvt_measure_pcie_both_ways": (_int, [_int, _u64, _u32, _P(C.c_double), _P(C.c_double)]),
    "kvt_copy_linear": (_int, [_vp, _vp, _u64, _vp]),
    "kvt_copy_runtime_d2d": (_int, [_vp, _vp, _u64, _vp]),
    "kvt_event_create": (_int, [_P(_vp)]),
    "kvt_event_destroy": (_int, [_vp]),
    "kvt_event_record": (_int, [_vp, _vp]),
    "kvt_event_synchronize": (_int, [_vp]),
    "kvt_event_elapsed_ms": (_int, [_vp, _vp, _P(C.c_float)]),
    "kvt_stream_create": (_int, [_P(_vp)]),
    "kvt_stream_destroy": (_int, [_vp]),
    "kvt_stream_synchronize": (_int, [_vp]),
}


class KvtError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("kvt error %d: %s" % (code, message))
        self.code = code


_lib = None


def _preload_hip_runtime():
    """A process must hold ONE HIP runtime. PyTorch wheels bundle their own
    libamdhip64 (same SONAME as the system one); if this library were loaded
    first it would bind the system runtime and a later ``import torch`` would
    bring in a second one that then finds no device. So when PyTorch is
    installed but not imported yet, its runtime is mapped first and the
    dynamic loader resolves this library's dependency to it by SONAME."""
    if "torch" in sys.modules:
        return
    try:
        spec = importlib.util.find_spec("torch")
    except (ImportError, ValueError):
        spec = None
    if spec is None or not spec.origin:
        return
    cand = os.path.join(os.path.dirname(spec.origin), "lib", "libamdhip64.so")
    if os.path.exists(cand):
        C.CDLL(cand, mode=C.RTLD_GLOBAL)


def lib():
    """Loads libkvt_hip.so (built in-tree by ``make -C llumnix-kv_amd``)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise KvtError(-1, "libkvt_hip.so is not built: run `make -C llumnix-kv_amd` "
                               "(or __graft_entry__.build())")
        _preload_hip_runtime()
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        _lib = handle
    return _lib


def _quiet_close(obj):
    """__del__ hook: at interpreter shutdown the module globals may already be gone."""
    try:
        obj.close()
    except Exception:
        pass


def check(rc):
    if rc != 0:
        raise KvtError(rc, (lib().kvt_last_error() or b"").decode())


def device_count():
    return lib().kvt_device_count()


def set_copy_cu_usage(device, usage):
    """Share of the device's CUs that copy launches may occupy (the reference's
    BLLM_KVTRANS_KERNEL_COPY_SM_USAGE, kvtransfer/src/envcfg.cpp:311-326); 1.0 = no limit."""
    check(lib().kvt_set_copy_cu_usage(device, float(usage)))


def get_copy_cu_usage(device):
    """-> (usage, workgroup limit; 0 = none)"""
    u, m = C.c_double(), _u32()
    check(lib().kvt_get_copy_cu_usage(device, C.byref(u), C.byref(m)))
    return u.value, m.value


def compute_valid_ranks_pd(p_tp, d_tp, heads):
    return lib().kvt_compute_valid_ranks_pd(p_tp, d_tp, heads)


def select_parser(cache_shape, src, dst):
    """-> (valid_mask, kvt_tp_size, kvt_tp_rank, parser_id, tp_kind)"""
    v, s, r, pid, kind = _u32(), _u32(), _u32(), _int(), _int()
    check(lib().kvt_select_parser(cache_shape, C.byref(src), C.byref(dst), C.byref(v), C.byref(s),
                                  C.byref(r), C.byref(pid), C.byref(kind)))
    return v.value, s.value, r.value, pid.value, kind.value


def merge_interval(runs):
    """runs: (n,3) uint64 -> (merged (m,3) array, (min,max,total,count))"""
    a = np.ascontiguousarray(runs, dtype=np.uint64).reshape(-1, 3).copy()
    n_out = _u64()
    stats = (_u64 * 4)()
    check(lib().kvt_merge_interval(a.ctypes.data, len(a), C.byref(n_out), stats))
    return a[:n_out.value].copy(), tuple(stats)


def wire_layout_of(fmt, lists):
    lay = WireLayout()
    check(lib().kvt_wire_layout_of(fmt, lists.h, C.byref(lay)))
    return lay


def wire_write_frame(fmt, buf_ptr, capacity, reqid, layer_idx, lists):
    lay = WireLayout()
    check(lib().kvt_wire_write_frame(fmt, buf_ptr, capacity, reqid, layer_idx, lists.h,
                                     C.byref(lay)))
    return lay


def wire_parse_frame(fmt, buf_ptr, length, expect_tensors=0):
    """-> (rc, reqid, layer_idx, BlockLists, WireLayout)"""
    lay, reqid, layer = WireLayout(), _u64(), _u64()
    lists = BlockLists()
    rc = lib().kvt_wire_parse_frame(fmt, buf_ptr, length, expect_tensors, C.byref(reqid),
                                    C.byref(layer), lists.h, C.byref(lay))
    return rc, reqid.value, layer.value, lists, lay


def block_object_lists(cache_shape, src, dst, src_blocks, dst_blocks, lists=None):
    """-> (BlockLists, object_bytes)"""
    lists = lists or BlockLists()
    s = np.ascontiguousarray(src_blocks, dtype=np.uint32)
    d = np.ascontiguousarray(dst_blocks, dtype=np.uint32)
    ob = _u64()
    check(lib().kvt_block_object_lists(cache_shape, C.byref(src), C.byref(dst), s.ctypes.data,
                                       d.ctypes.data, len(s), lists.h, C.byref(ob)))
    return lists, ob.value


def enlarge_block_ids(ids, factor):
    a = np.ascontiguousarray(ids, dtype=np.uint32)
    out = np.empty(len(a) * factor, dtype=np.uint32)
    check(lib().kvt_enlarge_block_ids(a.ctypes.data, len(a), factor, out.ctypes.data))
    return out


def validate_bounds(runs, capacity, which, scale=1):
    """-> (rc, bad_index)"""
    a = np.ascontiguousarray(runs, dtype=np.uint64).reshape(-1, 3)
    bad = _u64(0)
    rc = lib().kvt_validate_ipc_block_bounds(a.ctypes.data, len(a), capacity, which, scale,
                                             C.byref(bad))
    return rc, bad.value


class BlockLists:
    def __init__(self):
        self.h = _vp()
        check(lib().kvt_block_lists_create(C.byref(self.h)))

    def close(self):
        if self.h:
            lib().kvt_block_lists_destroy(self.h)
            self.h = _vp()

    __del__ = _quiet_close

    def clear(self):
        lib().kvt_block_lists_clear(self.h)

    def merge(self):
        check(lib().kvt_block_lists_merge(self.h))

    def num_tensors(self):
        return lib().kvt_block_lists_num_tensors(self.h)

    def append(self, t, runs):
        a = np.ascontiguousarray(runs, dtype=np.uint64).reshape(-1, 3)
        check(lib().kvt_block_lists_append(self.h, t, a.ctypes.data, len(a)))

    def tensor(self, t):
        """-> (n,3) uint64 copy of tensor t's ranges"""
        data = _P(IpcBlock)()
        n = _u64()
        check(lib().kvt_block_lists_view(self.h, t, C.byref(data), C.byref(n)))
        if n.value == 0:
            return np.zeros((0, 3), dtype=np.uint64)
        arr = np.ctypeslib.as_array(C.cast(data, _P(_u64)), shape=(n.value, 3))
        return arr.copy()

    def all(self):
        return [self.tensor(t) for t in range(self.num_tensors())]


class RunLists:
    """Per-tensor lists of strided runs (kvt_run, 11 uint64 words each)."""

    def __init__(self):
        self.h = _vp()
        check(lib().kvt_run_lists_create(C.byref(self.h)))

    def close(self):
        if self.h:
            lib().kvt_run_lists_destroy(self.h)
            self.h = _vp()

    __del__ = _quiet_close

    def clear(self):
        lib().kvt_run_lists_clear(self.h)

    def num_tensors(self):
        return lib().kvt_run_lists_num_tensors(self.h)

    def tensor(self, t):
        """-> structured copy of tensor t's runs"""
        data, n = _vp(), _u64()
        check(lib().kvt_run_lists_view(self.h, t, C.byref(data), C.byref(n)))
        if n.value == 0:
            return np.zeros(0, dtype=RUN_DTYPE)
        buf = (C.c_uint8 * (n.value * RUN_DTYPE.itemsize)).from_address(data.value)
        return np.frombuffer(buf, dtype=RUN_DTYPE).copy()

    def append(self, t, runs):
        """runs: structured array of RUN_DTYPE"""
        a = np.ascontiguousarray(runs, dtype=RUN_DTYPE)
        check(lib().kvt_run_lists_append(self.h, t, a.ctypes.data, len(a)))

    def totals(self, t):
        """-> (ranges, bytes) the runs of tensor t expand to"""
        a, b = _u64(), _u64()
        check(lib().kvt_run_lists_totals(self.h, t, C.byref(a), C.byref(b)))
        return a.value, b.value

    def expand(self, lists=None):
        lists = lists or BlockLists()
        check(lib().kvt_run_lists_expand(self.h, lists.h))
        return lists

    @staticmethod
    def compress(lists):
        out = RunLists()
        check(lib().kvt_run_lists_compress(lists.h, out.h))
        return out


CHUNK_DTYPE = np.dtype([("cache", "<u8"), ("packed", "<u8"), ("len", "<u4"), ("tensor", "<u2"),
                        ("t0", "<u2"), ("shape", "<u4"), ("reserved", "<u4")])
SHAPE_DTYPE = np.dtype([("vlen", "<u4"), ("inv_vlen", "<u4"), ("n_inner", "<u4"),
                        ("inv_wlen", "<u4"), ("outer", "<u8", 2), ("inner", "<u8", 2),
                        ("inv_inner", "<u4"), ("reserved", "<u4", 3)])
RUN_DTYPE = np.dtype([("src_offset", "<u8"), ("dst_offset", "<u8"), ("length", "<u8"),
                      ("n", "<u4", 3), ("reserved0", "<u4"), ("src_stride", "<u8", 3),
                      ("dst_stride", "<u8", 3)])


class Parser:
    def __init__(self, parser_id, src, dst, valid, tp_size, tp_rank, fp8=False, pad=True):
        self.h = _vp()
        opts = ParseOpts(1 if fp8 else 0, 1 if pad else 0)
        check(lib().kvt_parser_create(parser_id, C.byref(src), C.byref(dst), valid, tp_size,
                                      tp_rank, C.byref(opts), C.byref(self.h)))

    def close(self):
        if self.h:
            lib().kvt_parser_destroy(self.h)
            self.h = _vp()

    __del__ = _quiet_close

    def parse(self, task_struct, lists):
        """Appends one task's ranges; returns the KVT_* code (0 = ok)."""
        return lib().kvt_parse_block(self.h, C.byref(task_struct), lists.h)

    def parse_runs(self, task_struct, run_lists):
        """Same ranges in run form (one run per block segment)."""
        return lib().kvt_parse_block_runs(self.h, C.byref(task_struct), run_lists.h)


def _ptr(x):
    """device / host pointer of a torch tensor, numpy array, int or None"""
    if x is None:
        return None
    if isinstance(x, int):
        return x
    if hasattr(x, "data_ptr"):
        return x.data_ptr()
    if hasattr(x, "ctypes"):
        return x.ctypes.data
    raise TypeError(type(x))


class Cache:
    """Registered layer-tensor base pointers (layers[layer][tensor])."""

    def __init__(self, device, layers, capacity):
        n_layers, n_tensors = len(layers), len(layers[0])
        flat = (_vp * (n_layers * n_tensors))(*[_ptr(t) for l in layers for t in l])
        cap = (_u64 * n_tensors)(*capacity)
        self.h = _vp()
        self._keep = layers
        check(lib().kvt_cache_register(device, flat, n_layers, n_tensors, cap, C.byref(self.h)))

    def close(self):
        if self.h:
            lib().kvt_cache_destroy(self.h)
            self.h = _vp()

    __del__ = _quiet_close


class Plan:
    def __init__(self, device, lists, src_capacity, dst_capacity, xform=None, chunk_bytes=0,
                 objects=None, bf16_to_fp8=False):
        """objects = (object_bytes, object_stride): per-block objects spanning all layers.
        bf16_to_fp8 (RunLists parsed in that mode only): pack converts while it gathers."""
        n = lists.num_tensors()
        sc = (_u64 * max(1, n))(*src_capacity)
        dc = (_u64 * max(1, n))(*dst_capacity)
        xf = None
        if xform is not None:
            xf = C.byref(Xform(1, *xform))
        self.h = _vp()
        if objects is not None:
            check(lib().kvt_plan_create_objects(device, lists.h, sc, dc, objects[0], objects[1],
                                                chunk_bytes, C.byref(self.h)))
            return
        if isinstance(lists, RunLists):
            if xform is not None:
                raise ValueError("no layout transform for a plan made from runs")
            create = (lib().kvt_plan_create_runs_bf16_to_fp8 if bf16_to_fp8
                      else lib().kvt_plan_create_runs)
            check(create(device, lists.h, sc, dc, chunk_bytes, C.byref(self.h)))
            return
        if bf16_to_fp8:
            raise ValueError("a converting plan is made from RunLists (RunLists.compress for plain lists)")
        check(lib().kvt_plan_create(device, lists.h, sc, dc, xf, chunk_bytes, C.byref(self.h)))

    @property
    def num_strided_chunks(self):
        return lib().kvt_plan_num_strided_chunks(self.h)

    def host_tables(self):
        """Host-only plans (device=-1): -> (pack table, unpack table, chunk_bytes, shapes)."""
        chunks, shapes, n, cb = _vp(), _vp(), _u64(), _u32()
        check(lib().kvt_plan_host_tables(self.h, C.byref(chunks), C.byref(n), C.byref(cb),
                                         C.byref(shapes)))
        if n.value:
            buf = (C.c_uint8 * (2 * n.value * CHUNK_DTYPE.itemsize)).from_address(chunks.value)
            table = np.frombuffer(buf, dtype=CHUNK_DTYPE).copy()
        else:
            table = np.zeros(0, dtype=CHUNK_DTYPE)
        sbuf = (C.c_uint8 * (16 * SHAPE_DTYPE.itemsize)).from_address(shapes.value)
        return (table[:n.value], table[n.value:], cb.value,
                np.frombuffer(sbuf, dtype=SHAPE_DTYPE).copy())

    def close(self):
        if self.h:
            lib().kvt_plan_destroy(self.h)
            self.h = _vp()

    __del__ = _quiet_close

    def ready(self):
        check(lib().kvt_plan_ready(self.h))

    @property
    def layer_bytes(self):
        return lib().kvt_plan_layer_bytes(self.h)

    @property
    def num_chunks(self):
        return lib().kvt_plan_num_chunks(self.h)

    def tensor_bytes(self, t):
        return lib().kvt_plan_tensor_bytes(self.h, t)

    def tensor_offset(self, t):
        return lib().kvt_plan_tensor_offset(self.h, t)

    def pack(self, cache, first_layer, n_layers, packed, layer_stride, stream=None):
        check(lib().kvt_pack(self.h, cache.h, first_layer, n_layers, _ptr(packed), layer_stride,
                             _ptr(stream)))

    def unpack(self, cache, first_layer, n_layers, packed, layer_stride, stream=None):
        check(lib().kvt_unpack(self.h, cache.h, first_layer, n_layers, _ptr(packed), layer_stride,
                               _ptr(stream)))

    def pack_at(self, cache, first_layer, n_layers, base, layer_stride, blob_offsets, stream=None):
        offs = (_u64 * 8)(*blob_offsets)
        check(lib().kvt_pack_at(self.h, cache.h, first_layer, n_layers, _ptr(base), layer_stride,
                                offs, _ptr(stream)))

    def unpack_at(self, cache, first_layer, n_layers, base, layer_stride, blob_offsets,
                  stream=None):
        offs = (_u64 * 8)(*blob_offsets)
        check(lib().kvt_unpack_at(self.h, cache.h, first_layer, n_layers, _ptr(base), layer_stride,
                                  offs, _ptr(stream)))


class PlanSlot(Plan):
    """A plan at a fixed device address that takes a new batch per fill (kvt_plan_slot_*): what
    launches recorded into a hipGraph read, so that every replay moves the batch of its step.
    runs=True: filled with RunLists (strided entries; bf16_to_fp8: converting pack)."""

    def __init__(self, device, n_tensors, src_capacity, dst_capacity, max_entries, xform=None,
                 chunk_bytes=0, max_layer_bytes=0, runs=False, bf16_to_fp8=False):
        sc = (_u64 * n_tensors)(*src_capacity)
        dc = (_u64 * n_tensors)(*dst_capacity)
        self.h = _vp()
        self.runs = runs
        if runs:
            if xform is not None:
                raise ValueError("no layout transform for a slot made for runs")
            check(lib().kvt_plan_slot_create_runs(device, n_tensors, sc, dc, chunk_bytes,
                                                  1 if bf16_to_fp8 else 0, max_entries,
                                                  max_layer_bytes, C.byref(self.h)))
        else:
            xf = C.byref(Xform(1, *xform)) if xform is not None else None
            check(lib().kvt_plan_slot_create(device, n_tensors, sc, dc, xf, chunk_bytes,
                                             max_entries, max_layer_bytes, C.byref(self.h)))

    def fill(self, lists, stream=None):
        """The next batch (BlockLists, or RunLists for a slot made for runs), copied to the
        device on `stream` -> SlotLayout. Raises KvtError and leaves the slot as it was when
        the batch does not fit."""
        lay = SlotLayout()
        fn = lib().kvt_plan_slot_fill_runs if self.runs else lib().kvt_plan_slot_fill
        check(fn(self.h, lists.h, _ptr(stream), C.byref(lay)))
        return lay


def copy_ticket_stats(device):
    """-> (eager launches with a block of work counters, eager launches that found none,
    blocks handed to stream captures, captured launches that found none)"""
    out = (_u64 * 4)()
    check(lib().kvt_get_copy_ticket_stats(device, out))
    return tuple(out)


class Session:
    def __init__(self, plan, cache, packed, layer_stride):
        self.h = _vp()
        self._keep = (plan, cache, packed)
        check(lib().kvt_session_create(plan.h, cache.h, _ptr(packed), layer_stride,
                                       C.byref(self.h)))

    def close(self):
        if self.h:
            lib().kvt_session_destroy(self.h)
            self.h = _vp()

    __del__ = _quiet_close

    def save_layer(self, layer, compute_stream=None):
        check(lib().kvt_session_save_layer(self.h, layer, _ptr(compute_stream)))

    def save_layers(self, first_layer, n_layers, compute_stream=None):
        """Layers [first_layer, first_layer + n_layers) behind one event, packed by one launch."""
        check(lib().kvt_session_save_layers(self.h, first_layer, n_layers, _ptr(compute_stream)))

    def save_layers_inline(self, first_layer, n_layers, compute_stream=None):
        """The same on compute_stream itself: no hop to the side stream (a step's last layers)."""
        check(lib().kvt_session_save_layers_inline(self.h, first_layer, n_layers, _ptr(compute_stream)))

    def save_layer_event(self, layer, ready_event):
        """ready_event: a hipEvent_t handle the caller has recorded (an int, e.g.
        torch.cuda.Event.cuda_event), or the torch event itself."""
        handle = getattr(ready_event, "cuda_event", ready_event)
        check(lib().kvt_session_save_layer_event(self.h, layer, handle))

    def set_plan(self, plan, packed, layer_stride):
        """The next batch on the same session (its stream, events and counters are kept)."""
        check(lib().kvt_session_set_plan(self.h, plan.h, _ptr(packed), layer_stride))
        self._keep = (plan, self._keep[1], packed)

    def begin_step(self):
        """Starts the next step (host only; before each eager step, or before each launch of a
        graph that holds captured save_layer calls) -> its number."""
        step = _u64()
        check(lib().kvt_session_begin_step(self.h, C.byref(step)))
        return step.value

    def wait_layer(self, layer, step=0, timeout_us=None):
        """Blocks until `layer` of `step` (0 = the newest step) is packed; with timeout_us,
        raises KvtError(ERR_TIMEOUT) when that takes longer."""
        if timeout_us is None:
            check(lib().kvt_session_wait_layer_step(self.h, step, layer))
        else:
            check(lib().kvt_session_wait_layer_for(self.h, step, layer, int(timeout_us)))

    def join(self, stream=None):
        check(lib().kvt_session_join(self.h, _ptr(stream)))

    @property
    def side_stream(self):
        return lib().kvt_session_side_stream(self.h)


class Stager:
    def __init__(self, device, slot_bytes, n_slots):
        self.h = _vp()
        self.slot_bytes, self.n_slots = slot_bytes, n_slots
        check(lib().kvt_stager_create(device, slot_bytes, n_slots, C.byref(self.h)))

    def close(self):
        if self.h:
            lib().kvt_stager_destroy(self.h)
            self.h = _vp()

    __del__ = _quiet_close

    def slot_ptr(self, slot):
        return lib().kvt_stager_slot(self.h, slot)

    def slot_array(self, slot, nbytes):
        buf = (C.c_uint8 * nbytes).from_address(self.slot_ptr(slot))
        return np.frombuffer(buf, dtype=np.uint8)

    @property
    def copy_stream(self):
        return lib().kvt_stager_copy_stream(self.h)

    def save_at(self, slot, offset, dev, nbytes, producer_stream=None):
        check(lib().kvt_stager_save_at(self.h, slot, offset, _ptr(dev), nbytes,
                                       _ptr(producer_stream)))

    def load_at(self, slot, offset, dev, nbytes, consumer_stream=None):
        check(lib().kvt_stager_load_at(self.h, slot, offset, _ptr(dev), nbytes,
                                       _ptr(consumer_stream)))

    def save(self, slot, dev, nbytes, producer_stream=None):
        check(lib().kvt_stager_save(self.h, slot, _ptr(dev), nbytes, _ptr(producer_stream)))

    def load(self, slot, dev, nbytes, consumer_stream=None):
        check(lib().kvt_stager_load(self.h, slot, _ptr(dev), nbytes, _ptr(consumer_stream)))

    def wait(self, slot):
        check(lib().kvt_stager_wait(self.h, slot))


class ObjectRing:
    """Pinned ring of per-block store objects found by block hash (kvt_object_ring_*).
    Keys: bytes objects of `key_bytes` each."""

    def __init__(self, device, entry_bytes, n_entries, key_bytes):
        self.h = _vp()
        self.entry_bytes, self.n_entries, self.key_bytes = entry_bytes, n_entries, key_bytes
        check(lib().kvt_object_ring_create(device, entry_bytes, n_entries, key_bytes,
                                           C.byref(self.h)))

    def _keys(self, keys):
        assert all(len(k) == self.key_bytes for k in keys)
        return b"".join(keys)

    def reserve(self, keys):
        """-> (entries, is_new) as numpy arrays"""
        n = len(keys)
        e, f = np.zeros(n, dtype=np.uint32), np.zeros(n, dtype=np.uint8)
        check(lib().kvt_object_ring_reserve(self.h, self._keys(keys), n, e.ctypes.data,
                                            f.ctypes.data))
        return e, f.astype(bool)

    def lookup(self, keys):
        """-> (entries, found)"""
        n = len(keys)
        e, f = np.zeros(n, dtype=np.uint32), np.zeros(n, dtype=np.uint8)
        check(lib().kvt_object_ring_lookup(self.h, self._keys(keys), n, e.ctypes.data,
                                           f.ctypes.data))
        return e, f.astype(bool)

    def save(self, entries, dev_ptr, dev_stride, stream=None):
        e = np.ascontiguousarray(entries, dtype=np.uint32)
        check(lib().kvt_object_ring_save(self.h, e.ctypes.data, len(e), dev_ptr, dev_stride,
                                         stream))

    def load(self, entries, dev_ptr, dev_stride, stream=None, keys=None):
        """keys: the keys the entries were looked up with (checked against the entries)."""
        e = np.ascontiguousarray(entries, dtype=np.uint32)
        k = self._keys(keys) if keys is not None else None
        assert keys is None or len(keys) == len(e)
        check(lib().kvt_object_ring_load(self.h, e.ctypes.data, k, len(e), dev_ptr, dev_stride,
                                         stream))

    def release(self, entries):
        e = np.ascontiguousarray(entries, dtype=np.uint32)
        check(lib().kvt_object_ring_release(self.h, e.ctypes.data, len(e)))

    def commit(self, entries):
        e = np.ascontiguousarray(entries, dtype=np.uint32)
        check(lib().kvt_object_ring_commit(self.h, e.ctypes.data, len(e)))

    def wait(self, entry):
        check(lib().kvt_object_ring_wait(self.h, int(entry)))

    STATS = ("blocks_asked_for", "blocks_already_here", "entries_given_away", "lookups_found",
             "lookups_missed", "bytes_saved", "bytes_loaded", "entries_in_use")

    def stats(self):
        """-> dict of the ring's counters (kvt_object_ring_counters)."""
        out = (C.c_uint64 * len(self.STATS))()
        check(lib().kvt_object_ring_stats(self.h, out))
        return dict(zip(self.STATS, out))

    def entry(self, entry):
        """The entry's bytes as a numpy view of the ring's host memory."""
        p = lib().kvt_object_ring_entry(self.h, int(entry))
        if not p:
            raise IndexError(entry)
        return np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_uint8)), shape=(self.entry_bytes,))

    def close(self):
        if self.h:
            lib().kvt_object_ring_destroy(self.h)
            self.h = _vp()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
