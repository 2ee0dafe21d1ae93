"""kvt_adapter::LoopbackChannel (llumnix-kv_amd/adapter/kvt_loopback_channel.hpp) is a C++
implementation of the reference's IChannel (kvtransfer/include/channel.h:59-83) compiled
against the reference's own headers. oracle/adapter_check.cpp drives it through the
protocol KvSendStub uses -- connect, then per batch register_data / send_data(layer) for
every layer / flush -- and this test checks what landed in the receiver's paged cache
against the CPU oracle, bit for bit, plus the in-place merge and the metric string the
reference's channels produce. Needs a real MI355X and the checker built where the reference
checkout exists (`make -C oracle adapter`); skipped otherwise."""
import ctypes as C
import os

import numpy as np
import pytest

import checkers
import kvt_amd
from kvt_amd import workloads
from kvt_amd.ctypes_defs import IpcBlock
from test_gpu_pack import _host, _make_caches

SO = os.path.join(checkers.ROOT, "oracle", "_ref", "libkvt_adapter_check.so")
pytestmark = [pytest.mark.gpu,
              pytest.mark.skipif(not os.path.exists(SO), reason="adapter checker not built")]

torch = pytest.importorskip("torch")

ALLOC = C.CFUNCTYPE(C.c_void_p, C.c_size_t)
RELEASE = C.CFUNCTYPE(None, C.c_void_p)


class TorchBuffers:
    """The transfer buffer comes from the framework's allocator, as it would in an engine."""

    def __init__(self):
        self.live, self.allocs = {}, 0
        self.alloc = ALLOC(self._alloc)
        self.release = RELEASE(self._release)

    def _alloc(self, n):
        t = torch.empty(n, dtype=torch.uint8, device="cuda")
        self.live[t.data_ptr()] = t
        self.allocs += 1
        return t.data_ptr()

    def _release(self, p):
        del self.live[p]


def _lib():
    kvt_amd.lib()                      # maps the product library (and one HIP runtime) first
    lib = C.CDLL(SO)
    lib.kvtadp_loopback_send.argtypes = [
        C.c_int, C.POINTER(C.c_void_p), C.POINTER(C.c_uint64), C.POINTER(C.c_void_p),
        C.POINTER(C.c_uint64), C.c_uint32, C.c_uint32, C.POINTER(C.POINTER(IpcBlock)),
        C.POINTER(C.c_uint64), C.c_int, C.c_uint32, C.c_void_p, ALLOC, RELEASE, C.c_char_p,
        C.c_size_t]
    lib.kvtadp_loopback_send.restype = C.c_int
    return lib


def _send(w, lists, kind, batches=1, seed=5):
    """-> (rc, metrics dict or message, lists after register_data, src layers, dst layers, bufs)"""
    lib = _lib()
    n_t = w.n_tensors
    src_layers = _make_caches(w, "src", seed)
    dst_layers = _make_caches(w, "dst", seed + 1, fill=False)
    flat = lambda layers: (C.c_void_p * (w.n_layers * n_t))(*[t.data_ptr() for l in layers for t in l])
    s_cap = (C.c_uint64 * n_t)(*w.capacities("src"))
    d_cap = (C.c_uint64 * n_t)(*w.capacities("dst"))
    arrays = [np.ascontiguousarray(a, dtype=np.uint64).copy() for a in lists]
    ptrs = (C.POINTER(IpcBlock) * n_t)(*[C.cast(a.ctypes.data, C.POINTER(IpcBlock)) for a in arrays])
    counts = (C.c_uint64 * n_t)(*[len(a) for a in arrays])
    bufs = TorchBuffers()
    msg = C.create_string_buffer(512)
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.kvtadp_loopback_send(0, flat(src_layers), s_cap, flat(dst_layers), d_cap, w.n_layers,
                                  n_t, ptrs, counts, kind, batches, stream, bufs.alloc,
                                  bufs.release, msg, len(msg))
    torch.cuda.synchronize()
    text = msg.value.decode()
    after = [a[:counts[t]] for t, a in enumerate(arrays)]
    if rc == 0:
        text = dict(kv.split("=") for kv in text.strip(",").split(","))
    return rc, text, after, src_layers, dst_layers, bufs


def _expect_dst(w, runs_per_tensor, src_layers, dst_layers):
    for l in range(w.n_layers):
        for t in range(w.n_tensors):
            blob = checkers.oracle_pack(_host(src_layers[l][t]), runs_per_tensor[t])
            exp = np.full(w.capacities("dst")[t], 0xA5, dtype=np.uint8)
            checkers.oracle_unpack(exp, runs_per_tensor[t], blob)
            assert np.array_equal(_host(dst_layers[l][t]), exp), (l, t)


def _oracle_unmerged(w):
    src, dst = w.worker_infos()
    rc, valid, tps, tpr, pid, kind = checkers.oracle_select(w.cache_shape, src, dst)
    assert rc == 0
    rc, outs = checkers.oracle_parse(pid, src, dst, valid, tps, tpr, w.task_bufs())
    assert rc == 0
    return outs, kind


def test_p_eq_d_batch_is_merged_in_place_and_lands_in_the_receivers_cache():
    w = workloads.deepseek_mla(n_layers=3, pool=96, n_req=3, tokens=1500)     # two tensors per layer
    outs, kind = _oracle_unmerged(w)
    assert kind == 0
    rc, m, after, src_layers, dst_layers, bufs = _send(w, outs, kind, batches=2)
    assert rc == 0, m
    merged = [checkers.oracle_merge(o) for o in outs]
    for t in range(w.n_tensors):
        assert np.array_equal(after[t], merged[t][0])                       # register_data's in-place merge
    _expect_dst(w, [mm[0] for mm in merged], src_layers, dst_layers)
    assert int(m["OriginSbNum"]) == sum(len(o) for o in outs)
    assert int(m["MergedSbNum"]) == sum(len(mm[0]) for mm in merged)
    assert int(m["SbSizeMin"]) == min(mm[1][0] for mm in merged)
    assert int(m["SbSizeMax"]) == max(mm[1][1] for mm in merged)
    assert int(m["SbSizeTotal"]) == sum(int(mm[0][:, 2].sum()) for mm in merged)
    assert int(m["LayersSent"]) == w.n_layers and m["closed"] == "1"
    assert bufs.allocs == 1 and not bufs.live          # one transfer buffer served both batches


def test_tp_remapping_batch_goes_through_strided_records():
    w = workloads.tp_split("flash", 2, 1, 1, n_layers=2, src_pool=300, dst_pool=400, n_req=4,
                           min_tok=100, max_tok=900)
    outs, kind = _oracle_unmerged(w)
    assert kind == 2                                    # TPKind::PGTD: sent as parsed, never merged
    rc, m, after, src_layers, dst_layers, _ = _send(w, outs, kind)
    assert rc == 0, m
    assert np.array_equal(after[0], outs[0])
    _expect_dst(w, outs, src_layers, dst_layers)
    assert int(m["OriginSbNum"]) == int(m["MergedSbNum"]) == len(outs[0])


def test_receiver_refuses_a_range_outside_its_cache_like_the_reference():
    w = workloads.llama8b_batch(n_layers=2, src_pool=128, dst_pool=192, n_req=2, min_tok=100,
                                max_tok=400)
    outs, kind = _oracle_unmerged(w)
    bad = outs[0].copy()
    bad[3, 1] = w.capacities("dst")[0] - 16             # the range now runs off the destination
    rc, text, _, _, dst_layers, bufs = _send(w, [bad], kind)
    assert rc == 1, text                                # std::out_of_range, as channel.cpp:11-50 throws
    assert not bufs.live
    for l in range(w.n_layers):
        assert (_host(dst_layers[l][0]) == 0xA5).all()  # nothing was scattered
