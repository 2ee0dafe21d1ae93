"""Plan slots checked without a GPU (kvt_plan_slot_*): a host-only slot (device = -1) keeps the
tables of its newest fill on the host; refilled with batch after batch -- different block
tables, request counts, an empty batch, one that takes every entry -- each fill's tables,
walked with the kernels' addressing (test_plan_tables.emulate), must reproduce the CPU oracle's
pack / unpack of THAT batch, and a batch that does not fit is refused with the slot unchanged.
The reference builds a new range list per batch (kvtransfer/src/tx_stub.cpp:158-263)."""
import numpy as np
import pytest

import checkers
import kvt_amd
from kvt_amd import pipeline, workloads
from test_plan_tables import _check_tables, _oracle_ranges


def _batches():
    """Config-2-shaped batches of different sizes on the same pools."""
    out = []
    for seed, n_req, hi in ((1, 5, 200), (2, 1, 40), (3, 9, 120), (4, 3, 330)):
        out.append(workloads.llama8b_batch(n_layers=1, src_pool=96, dst_pool=128, n_req=n_req,
                                           min_tok=10, max_tok=hi, seed=seed))
    return out


def _lists(w):
    src, dst = w.worker_infos()
    lists, _ = pipeline.parse_batch(w.cache_shape, src, dst, w.task_bufs())
    return lists


@pytest.mark.parametrize("chunk", [0, 4096, 8192, 16384])
def test_refills_give_the_tables_of_a_fresh_plan(chunk):
    ws = _batches()
    s_cap, d_cap = ws[0].capacities("src"), ws[0].capacities("dst")
    slot = kvt_amd.PlanSlot(-1, 1, s_cap, d_cap, max_entries=4096, chunk_bytes=chunk)
    for k, w in enumerate(ws):
        lists = _lists(w)
        lay = slot.fill(lists)
        fresh = kvt_amd.Plan(-1, lists, s_cap, d_cap, chunk_bytes=chunk or 32768)
        assert lay.n_entries == slot.num_chunks == fresh.num_chunks
        assert lay.layer_bytes == slot.layer_bytes == fresh.layer_bytes
        assert lay.tensor_bytes[0] == fresh.tensor_bytes(0)
        assert lay.tensor_offset[0] == fresh.tensor_offset(0)
        a, b = slot.host_tables(), fresh.host_tables()
        assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1]) and a[2] == b[2]
        _check_tables(slot, _oracle_ranges(w), s_cap, d_cap, 40 + k)


def test_an_empty_batch_and_one_that_takes_every_entry():
    w = _batches()[0]
    s_cap, d_cap = w.capacities("src"), w.capacities("dst")
    lists = _lists(w)
    need = kvt_amd.Plan(-1, lists, s_cap, d_cap, chunk_bytes=32768).num_chunks
    slot = kvt_amd.PlanSlot(-1, 1, s_cap, d_cap, max_entries=need)
    assert slot.fill(lists).n_entries == need                    # at capacity
    _check_tables(slot, _oracle_ranges(w), s_cap, d_cap, 5)
    for empty in (kvt_amd.BlockLists(), None):
        if empty is None:                                        # one tensor, no ranges
            empty = kvt_amd.BlockLists()
            empty.append(0, np.zeros((0, 3), dtype=np.uint64))
        lay = slot.fill(empty)
        assert (lay.n_entries, lay.layer_bytes, lay.tensor_bytes[0]) == (0, 0, 0)
        assert slot.num_chunks == 0 and len(slot.host_tables()[0]) == 0
    assert slot.fill(lists).n_entries == need


def test_a_batch_that_does_not_fit_is_refused_and_the_slot_keeps_its_contents():
    ws = _batches()
    s_cap, d_cap = ws[0].capacities("src"), ws[0].capacities("dst")
    small, large = _lists(ws[1]), _lists(ws[2])
    n_small = kvt_amd.Plan(-1, small, s_cap, d_cap, chunk_bytes=32768).num_chunks
    n_large = kvt_amd.Plan(-1, large, s_cap, d_cap, chunk_bytes=32768).num_chunks
    assert n_small < n_large
    slot = kvt_amd.PlanSlot(-1, 1, s_cap, d_cap, max_entries=n_large - 1)
    slot.fill(small)
    before = [t.copy() for t in slot.host_tables()[:2]]
    with pytest.raises(kvt_amd.KvtError) as e:
        slot.fill(large)
    assert e.value.code == kvt_amd.ctypes_defs.ERR_OUT_OF_RANGE and "table entries" in str(e.value)
    after = slot.host_tables()
    assert np.array_equal(before[0], after[0]) and np.array_equal(before[1], after[1])
    assert slot.num_chunks == n_small
    # too many bytes for the room of a packed layer
    tight = kvt_amd.PlanSlot(-1, 1, s_cap, d_cap, max_entries=4096,
                             max_layer_bytes=kvt_amd.Plan(-1, large, s_cap, d_cap).layer_bytes - 256)
    tight.fill(small)
    with pytest.raises(kvt_amd.KvtError) as e:
        tight.fill(large)
    assert e.value.code == kvt_amd.ctypes_defs.ERR_OUT_OF_RANGE and "packed layer" in str(e.value)
    # ranges beyond the capacities the slot was made with
    with pytest.raises(kvt_amd.KvtError) as e:
        kvt_amd.PlanSlot(-1, 1, [s_cap[0] // 4], d_cap, max_entries=4096).fill(large)
    assert e.value.code == kvt_amd.ctypes_defs.ERR_OUT_OF_RANGE
    # a slot moves whole 16-byte vectors
    odd = kvt_amd.BlockLists()
    odd.append(0, [(0, 0, 4096), (8192, 8200, 100)])
    with pytest.raises(kvt_amd.KvtError) as e:
        slot.fill(odd)
    assert e.value.code == kvt_amd.ctypes_defs.ERR_INVALID and "16-byte" in str(e.value)
    assert slot.num_chunks == n_small
    # the wrong number of tensors, the wrong kind of list
    two = kvt_amd.BlockLists()
    two.append(1, [(0, 0, 4096)])
    with pytest.raises(kvt_amd.KvtError):
        slot.fill(two)
    with pytest.raises(kvt_amd.KvtError):
        kvt_amd.binding.check(kvt_amd.lib().kvt_plan_slot_fill_runs(slot.h, kvt_amd.RunLists().h, None, None))
    with pytest.raises(kvt_amd.KvtError):      # a plan made for one batch is no slot
        plain = kvt_amd.Plan(-1, small, s_cap, d_cap)
        kvt_amd.binding.check(kvt_amd.lib().kvt_plan_slot_fill(plain.h, small.h, None, None))


def test_slot_creation_checks_its_arguments():
    cap = [1 << 20]
    for kw in (dict(max_entries=0), dict(max_entries=1 << 27), dict(max_entries=8, chunk_bytes=5000),
               dict(max_entries=8, chunk_bytes=65536), dict(max_entries=8, chunk_bytes=2048)):
        with pytest.raises(kvt_amd.KvtError):
            kvt_amd.PlanSlot(-1, 1, cap, cap, **kw)
    with pytest.raises(kvt_amd.KvtError):
        kvt_amd.PlanSlot(-1, 0, [], [], max_entries=8)
    kvt_amd.PlanSlot(-1, 1, cap, cap, max_entries=8, chunk_bytes=65536, runs=True).close()


def test_two_tensors_per_layer_follow_the_batch():
    """The sparse-MLA layout: both tensors' blob positions move with the batch."""
    s_cap = d_cap = None
    slot = None
    for k, (n_req, tokens) in enumerate(((3, 700), (1, 90), (4, 300))):
        w = workloads.deepseek_mla(n_layers=1, pool=64, n_req=n_req, tokens=tokens)
        if slot is None:
            s_cap, d_cap = w.capacities("src"), w.capacities("dst")
            slot = kvt_amd.PlanSlot(-1, 2, s_cap, d_cap, max_entries=2048, chunk_bytes=4096)
        lists = _lists(w)
        lay = slot.fill(lists)
        fresh = kvt_amd.Plan(-1, lists, s_cap, d_cap, chunk_bytes=4096)
        for t in range(2):
            assert lay.tensor_bytes[t] == fresh.tensor_bytes(t)
            assert lay.tensor_offset[t] == fresh.tensor_offset(t)
        _check_tables(slot, _oracle_ranges(w), s_cap, d_cap, 60 + k)


@pytest.mark.parametrize("chunk", [0, 4096, 65536])
@pytest.mark.parametrize("layout,p_tp,d_tp,rank", [("flash", 2, 1, 1), ("ragged", 1, 2, 1),
                                                   ("hnd", 2, 1, 1)])
def test_run_slots_for_tp_split_batches(layout, p_tp, d_tp, rank, chunk):
    slot, caps = None, None
    for k, (n_req, hi) in enumerate(((4, 150), (1, 30), (6, 90))):
        w = workloads.tp_split(layout, p_tp, d_tp, rank, n_layers=1, src_pool=40, dst_pool=60,
                               n_req=n_req, min_tok=5, max_tok=hi, total_heads=4, head_dim=32,
                               seed=70 + k)
        src, dst = w.worker_infos()
        runs, _ = pipeline.parse_batch_runs(w.cache_shape, src, dst, w.task_bufs())
        if slot is None:
            caps = (w.capacities("src"), w.capacities("dst"))
            slot = kvt_amd.PlanSlot(-1, 1, caps[0], caps[1], max_entries=8192, chunk_bytes=chunk,
                                    runs=True)
        lay = slot.fill(runs)
        fresh = kvt_amd.Plan(-1, runs, caps[0], caps[1], chunk_bytes=chunk or 32768)
        assert lay.n_entries == fresh.num_chunks and slot.num_strided_chunks == fresh.num_strided_chunks
        a, b = slot.host_tables(), fresh.host_tables()
        assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
        n_shapes = int((b[3]["vlen"] != 0).sum())
        assert np.array_equal(a[3][:n_shapes], b[3][:n_shapes])
        _check_tables(slot, _oracle_ranges(w), caps[0], caps[1], 80 + k)
