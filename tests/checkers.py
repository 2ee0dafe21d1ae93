"""Loaders for the CPU checkers (test infrastructure only).

* ``oracle()``  -> oracle/libkvt_oracle.so, this repository's CPU restatement.
* ``ref()``     -> oracle/_ref/libkvt_ref.so, the reference's own ParseBlock
  sources compiled by ``make -C oracle ref``; ``None`` where it was never built
  (it can only be built where the reference checkout exists).
"""
import ctypes as C
import os
import subprocess

import numpy as np

from kvt_amd.ctypes_defs import IpcBlock, ParseOpts, Task, WorkerInfo, task_array

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_SO = os.path.join(ROOT, "oracle", "libkvt_oracle.so")
REF_SO = os.path.join(ROOT, "oracle", "_ref", "libkvt_ref.so")

_cache = {}

_PARSE_TAIL = [C.POINTER(Task), C.c_uint32, C.c_uint32, C.POINTER(C.POINTER(IpcBlock)),
               C.POINTER(C.c_uint64), C.POINTER(C.c_uint32)]
_PARSE_HEAD = [C.c_int, C.POINTER(WorkerInfo), C.POINTER(WorkerInfo), C.c_uint32, C.c_uint32,
               C.c_uint32]


def oracle():
    if "o" not in _cache:
        if not os.path.exists(ORACLE_SO):
            subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "oracle"])
        lib = C.CDLL(ORACLE_SO)
        lib.kvto_parse.argtypes = _PARSE_HEAD + [C.POINTER(ParseOpts)] + _PARSE_TAIL
        lib.kvto_parse.restype = C.c_int
        lib.kvto_free.argtypes = [C.c_void_p]
        lib.kvto_valid_ranks.argtypes = [C.c_uint32, C.c_uint32, C.c_int]
        lib.kvto_valid_ranks.restype = C.c_uint32
        lib.kvto_select.argtypes = [C.c_int, C.POINTER(WorkerInfo), C.POINTER(WorkerInfo),
                                    C.POINTER(C.c_uint32), C.POINTER(C.c_uint32),
                                    C.POINTER(C.c_uint32), C.POINTER(C.c_int), C.POINTER(C.c_int)]
        lib.kvto_select.restype = C.c_int
        lib.kvto_merge.argtypes = [C.c_void_p, C.c_uint64, C.POINTER(C.c_uint64)]
        lib.kvto_merge.restype = C.c_uint64
        lib.kvto_validate.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64, C.c_int, C.c_uint64,
                                      C.POINTER(C.c_uint64)]
        lib.kvto_validate.restype = C.c_int
        for name in ("kvto_pack", "kvto_unpack", "kvto_pack_bf16_to_fp8"):
            getattr(lib, name).argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_void_p]
            getattr(lib, name).restype = None
        for name in ("kvto_pack_layers", "kvto_unpack_layers"):
            getattr(lib, name).argtypes = [C.c_void_p, C.c_uint32, C.c_void_p, C.c_uint64,
                                           C.c_void_p, C.c_uint64, C.c_uint32]
            getattr(lib, name).restype = None
        for name in ("kvto_pack_hnd_to_nhd", "kvto_unpack_nhd_to_hnd"):
            getattr(lib, name).argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_uint32,
                                           C.c_uint32, C.c_uint32, C.c_void_p]
            getattr(lib, name).restype = None
        lib.kvto_bf16_to_fp8.argtypes = [C.c_uint16]
        lib.kvto_bf16_to_fp8.restype = C.c_uint8
        _cache["o"] = lib
    return _cache["o"]


def ref():
    if "r" not in _cache:
        lib = None
        if os.path.exists(REF_SO):
            lib = C.CDLL(REF_SO)
            lib.kvtref_parse.argtypes = _PARSE_HEAD + _PARSE_TAIL
            lib.kvtref_parse.restype = C.c_int
            lib.kvtref_free.argtypes = [C.c_void_p]
            lib.kvtref_plan_parse.argtypes = _PARSE_HEAD + _PARSE_TAIL + [C.POINTER(C.c_int)]
            lib.kvtref_plan_parse.restype = C.c_int
        _cache["r"] = lib
    return _cache["r"]


def _collect(free, outs, n_out, n_tensors, cap):
    res = []
    for t in range(min(n_tensors, cap)):
        n = n_out[t]
        arr = np.ctypeslib.as_array(C.cast(outs[t], C.POINTER(C.c_uint64)), shape=(max(n, 1), 3))
        res.append(arr[:n].copy())
        free(outs[t])
    return res


def _run(fn, free, head, tasks, extra, tail=()):
    cap = 8
    outs = (C.POINTER(IpcBlock) * cap)()
    n_out = (C.c_uint64 * cap)()
    n_t = C.c_uint32(0)
    arr = task_array(tasks)
    rc = fn(*head, *extra, arr, len(tasks), cap, outs, n_out, C.byref(n_t), *tail)
    if rc != 0:
        return rc, []
    return rc, _collect(free, outs, n_out, n_t.value, cap)


def oracle_parse(parser_id, src, dst, valid, tp_size, tp_rank, tasks, fp8=False, pad=True):
    """-> (rc, [per-tensor (n,3) uint64 arrays of (src_offset, dst_offset, length)])"""
    lib = oracle()
    opts = ParseOpts(1 if fp8 else 0, 1 if pad else 0)
    head = (parser_id, C.byref(src), C.byref(dst), valid, tp_size, tp_rank)
    return _run(lib.kvto_parse, lib.kvto_free, head, tasks, (C.byref(opts),))


def ref_parse(parser_id, src, dst, valid, tp_size, tp_rank, tasks):
    lib = ref()
    head = (parser_id, C.byref(src), C.byref(dst), valid, tp_size, tp_rank)
    return _run(lib.kvtref_parse, lib.kvtref_free, head, tasks, ())


def ref_plan_parse(cache_shape, src, dst, valid, tp_size, tp_rank, tasks):
    """The reference's descriptor-driven generator (cache_transfer_spec.cpp) on the same
    inputs -> (rc, per-tensor arrays, TPKind)."""
    lib = ref()
    kind = C.c_int(-1)
    head = (cache_shape, C.byref(src), C.byref(dst), valid, tp_size, tp_rank)
    rc, out = _run(lib.kvtref_plan_parse, lib.kvtref_free, head, tasks, (), (C.byref(kind),))
    return rc, out, kind.value


def oracle_select(shape, src, dst):
    lib = oracle()
    v, s, r = C.c_uint32(), C.c_uint32(), C.c_uint32()
    pid, kind = C.c_int(), C.c_int()
    rc = lib.kvto_select(shape, C.byref(src), C.byref(dst), C.byref(v), C.byref(s), C.byref(r),
                         C.byref(pid), C.byref(kind))
    return rc, v.value, s.value, r.value, pid.value, kind.value


def oracle_merge(runs):
    """runs: (n,3) uint64 -> (merged (m,3) array, (min,max,total,count))"""
    lib = oracle()
    a = np.ascontiguousarray(runs, dtype=np.uint64).copy()
    stats = (C.c_uint64 * 4)()
    m = lib.kvto_merge(a.ctypes.data, len(a), stats)
    return a[:m].copy(), tuple(stats)


def oracle_pack(layer, runs):
    lib = oracle()
    runs = np.ascontiguousarray(runs, dtype=np.uint64)
    out = np.empty(int(runs[:, 2].sum()) if len(runs) else 0, dtype=np.uint8)
    lib.kvto_pack(layer.ctypes.data, runs.ctypes.data, len(runs), out.ctypes.data)
    return out


def oracle_unpack(layer, runs, blob):
    lib = oracle()
    runs = np.ascontiguousarray(runs, dtype=np.uint64)
    lib.kvto_unpack(layer.ctypes.data, runs.ctypes.data, len(runs), blob.ctypes.data)


# ---------------------------------------------------------------- dispatch

# (prefix of the parser name, cache shape): which cache shape a parser id belongs to in the
# reference's per-destination dispatch (refresh_dst_info, kvtransfer/src/tx_stub.cpp:451-590)
_PARSER_SHAPES = (("RAGGED_", 1), ("FLASHINFER_", 5), ("FLASH_", 2), ("HYBRID_FI_", 7),
                  ("HYBRID_", 3), ("DPSK_", 4), ("KIMI_K3_", 8), ("TURBOQUANT_", 6))
_KIND_OF_SUFFIX = {"PEQD": 0, "PLTD": 1, "PGTD": 2}


def dispatch_of(parser_name):
    """-> (cache shape, TPKind) the reference's dispatch pairs with this parser, or None for
    the parsers it never selects directly (the KDA state parsers are called by the Kimi-K3
    ones). TPKind follows the name except where tx_stub.cpp says otherwise: every DPSK parser
    and parse_block_send_p_gt_d_dpsk are registered as PEQD (tx_stub.cpp:469-470, 521-535)."""
    for prefix, shape in _PARSER_SHAPES:
        if parser_name.startswith(prefix):
            if shape == 4 or parser_name == "RAGGED_PGTD_DPSK":
                return shape, 0
            return shape, _KIND_OF_SUFFIX[parser_name.rsplit("_", 1)[1]]
    return None


def assert_dispatch(parser_name, src, dst, valid=None, tp_size=None, tp_rank=None):
    """A known-answer case names its parser and its (valid ranks, kvt_tp_size, kvt_tp_rank):
    from (cache shape, src, dst) alone, the oracle's and the product's dispatch must arrive at
    exactly those. valid = None: the case hands the parser rank values it did not derive from
    the two workers (some reference tests do); then only parser and TPKind are compared."""
    from kvt_amd.ctypes_defs import PARSER
    import kvt_amd
    want = dispatch_of(parser_name)
    if want is None:     # never selected by the dispatch itself: nothing to check
        return
    shape, kind = want
    exp = (valid, tp_size, tp_rank, PARSER[parser_name], kind)
    got_o = oracle_select(shape, src, dst)
    got_p = kvt_amd.select_parser(shape, src, dst)
    if valid is None:
        exp, got_o, got_p = exp[3:], (got_o[0],) + got_o[4:], got_p[3:]
    assert got_o == (0,) + exp, ("oracle dispatch", parser_name, got_o, exp)
    assert got_p == exp, ("product dispatch", parser_name, got_p, exp)


def side_stream():
    """A stream of its own for a GPU test. The device is synchronized first: what the test has
    queued on torch's default stream so far (fills, seeded contents) is not ordered against
    work on any other stream, and a launch there could otherwise overtake it."""
    import torch
    torch.cuda.synchronize()
    return torch.cuda.Stream()
