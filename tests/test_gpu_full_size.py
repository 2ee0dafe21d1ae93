"""Full-size GPU checks of the benchmark configurations (2, 3, 4, 5) against an
implementation that shares nothing with the HIP kernels: the CPU oracle's
range lists turned into a 16-byte-unit index vector, and torch's own
index_select / index_copy (and permute for the HND<->NHD transform) doing the
gather and scatter on the GPU. Every layer is compared in full with
torch.equal. Needs a real MI355X with ~130 GiB of free HBM."""
import numpy as np
import pytest

import checkers
import kvt_amd
from kvt_amd import pipeline, workloads

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(autouse=True)
def _release_hbm():
    yield
    torch.cuda.empty_cache()     # hand the tens of GiB back before the next test allocates


def _oracle_lists(w):
    src, dst = w.worker_infos()
    rc, valid, tps, tpr, pid, kind = checkers.oracle_select(w.cache_shape, src, dst)
    assert rc == 0
    rc, outs = checkers.oracle_parse(pid, src, dst, valid, tps, tpr, w.task_bufs())
    assert rc == 0
    if kind == 0:
        outs = [checkers.oracle_merge(o)[0] for o in outs]
    return outs


def _unit_index(offsets, lengths):
    """16-byte-unit indices covered by the ranges, in list order (numpy int64)."""
    assert (offsets % 16 == 0).all() and (lengths % 16 == 0).all()
    starts = (offsets // 16).astype(np.int64)
    counts = (lengths // 16).astype(np.int64)
    first = np.cumsum(counts) - counts
    return np.repeat(starts - first, counts) + np.arange(int(counts.sum()), dtype=np.int64)


_SLICE = 1 << 24   # torch's index kernels refuse launches beyond ~2^26 rows: go in slices


def _gathered_equals(rows, idx, blob):
    """blob == rows[idx], compared slice by slice."""
    for a in range(0, len(idx), _SLICE):
        if not torch.equal(blob[a:a + _SLICE], rows.index_select(0, idx[a:a + _SLICE])):
            return False
    return True


def _scatter(exp_rows, idx, values):
    for a in range(0, len(idx), _SLICE):
        exp_rows.index_copy_(0, idx[a:a + _SLICE], values[a:a + _SLICE])


def _caches(w, seed):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    src, dst = [], []
    for l in range(w.n_layers):
        src.append([torch.randint(0, 256, (c,), generator=g, device="cuda", dtype=torch.uint8)
                    for c in w.capacities("src")])
        dst.append([torch.full((c,), 0xA5, device="cuda", dtype=torch.uint8)
                    for c in w.capacities("dst")])
    return src, dst


def _run_plain(w, seed, earlier=None, chunk=0):
    """earlier: another batch on the same pools. The plan then is a plan slot that held that
    batch first and was refilled with w's (kvt_plan_slot_fill), launched through the persistent
    kernels that read the batch's entry count and blob positions from the slot's header.
    chunk: the size the slot's table entries are cut to."""
    plan, lists = pipeline.build_plan(w, 0, chunk)
    o_lists = _oracle_lists(w)
    for t in range(w.n_tensors):
        assert np.array_equal(lists.tensor(t), o_lists[t])
    if earlier is not None:
        fresh = plan
        old_plan, old_lists = pipeline.build_plan(earlier, 0, chunk)
        room = max(fresh.layer_bytes, old_plan.layer_bytes)   # a layer's stride holds any batch of the slot
        plan = kvt_amd.PlanSlot(0, w.n_tensors, w.capacities("src"), w.capacities("dst"),
                                max_entries=max(fresh.num_chunks, old_plan.num_chunks),
                                max_layer_bytes=room, chunk_bytes=chunk)
        assert plan.fill(old_lists).n_entries == old_plan.num_chunks
        lay = plan.fill(lists)
        assert (lay.n_entries, lay.layer_bytes) == (fresh.num_chunks, fresh.layer_bytes)
        for t in range(w.n_tensors):
            assert (lay.tensor_bytes[t], lay.tensor_offset[t]) == (fresh.tensor_bytes(t), fresh.tensor_offset(t))
        old_plan.close()
        fresh.close()
    src, dst = _caches(w, seed)
    sc = kvt_amd.Cache(0, src, w.capacities("src"))
    dc = kvt_amd.Cache(0, dst, w.capacities("dst"))
    stride = plan.layer_bytes if earlier is None else room
    packed = torch.zeros(w.n_layers * stride, dtype=torch.uint8, device="cuda")
    plan.pack(sc, 0, w.n_layers, packed, stride)
    plan.unpack(dc, 0, w.n_layers, packed, stride)
    torch.cuda.synchronize()
    for t in range(w.n_tensors):
        runs = o_lists[t]
        s_idx = torch.from_numpy(_unit_index(runs[:, 0], runs[:, 2])).cuda()
        d_idx = torch.from_numpy(_unit_index(runs[:, 1], runs[:, 2])).cuda()
        assert len(torch.unique(d_idx)) == len(d_idx)          # the scatter is race-free
        nb = int(runs[:, 2].sum())
        assert plan.tensor_bytes(t) == nb
        off = plan.tensor_offset(t)
        for l in range(w.n_layers):
            blob = packed[l * stride + off: l * stride + off + nb].view(-1, 16)
            assert _gathered_equals(src[l][t].view(-1, 16), s_idx, blob), ("pack", l, t)
            exp = torch.full_like(dst[l][t], 0xA5).view(-1, 16)
            _scatter(exp, d_idx, blob)      # blob == the gathered source rows (just checked)
            assert torch.equal(dst[l][t].view(-1, 16), exp), ("unpack", l, t)
            del exp
    return plan


def test_config2_full_size():
    w = workloads.llama8b_batch()         # 64 requests x 1k-8k tokens, 32 layers, 34 GiB payload
    plan = _run_plain(w, 2)
    assert plan.layer_bytes * w.n_layers > 30 * 2**30


def test_config4_full_size():
    _run_plain(workloads.deepseek_mla(), 4)        # 61 layers, MLA latent + indexer, 10.5 GiB


def test_config2_full_size_through_a_refilled_plan_slot():
    w = workloads.llama8b_batch()
    _run_plain(w, 12, earlier=workloads.llama8b_batch(seed=4711), chunk=32768)


def test_config4_full_size_through_a_refilled_plan_slot():
    # two tensors per layer, entries of 4 KiB: a wavefront per entry
    _run_plain(workloads.deepseek_mla(), 14, earlier=workloads.deepseek_mla(n_req=9, tokens=9000), chunk=4096)


def test_config5_full_size():
    _run_plain(workloads.qwen3next_attn(), 5)      # 128 requests x 256 pages x 12 layers
    torch.cuda.empty_cache()
    _run_plain(workloads.qwen3next_gdn(), 6)       # 128 states of 2 MiB x 36 layers


def test_config3_full_size_transposing_pack():
    w = workloads.llama70b_flashinfer()            # 80 layers, 32 requests x 256 pages, 40 GiB
    heads, ntpb, row = w.xform
    plan, lists = pipeline.build_plan(w, 0)
    runs = _oracle_lists(w)[0]
    assert np.array_equal(lists.tensor(0), runs)
    B = 2 * heads * ntpb * row
    s_ids = torch.from_numpy(np.concatenate(
        [np.arange(r[0] // B, (r[0] + r[2]) // B) for r in runs]).astype(np.int64)).cuda()
    d_ids = torch.from_numpy(np.concatenate(
        [np.arange(r[1] // B, (r[1] + r[2]) // B) for r in runs]).astype(np.int64)).cuda()
    assert len(torch.unique(d_ids)) == len(d_ids)
    stride = plan.layer_bytes
    assert stride == len(s_ids) * B
    step = 8                                        # layers resident at a time
    g = torch.Generator(device="cuda")
    g.manual_seed(3)
    cap = w.capacities("src")[0]
    nblk = cap // B
    for first in range(0, w.n_layers, step):
        src = [[torch.randint(0, 256, (cap,), generator=g, device="cuda", dtype=torch.uint8)]
               for _ in range(step)]
        dst = [[torch.full((cap,), 0xA5, device="cuda", dtype=torch.uint8)] for _ in range(step)]
        sc, dc = kvt_amd.Cache(0, src, [cap]), kvt_amd.Cache(0, dst, [cap])
        packed = torch.zeros(step * stride, dtype=torch.uint8, device="cuda")
        plan.pack(sc, 0, step, packed, stride)
        plan.unpack(dc, 0, step, packed, stride)
        torch.cuda.synchronize()
        for l in range(step):
            hnd = src[l][0].view(nblk, 2, heads, ntpb, row)
            picked = hnd.index_select(0, s_ids)                                     # 8192 pages
            want = picked.permute(0, 1, 3, 2, 4).contiguous()                       # -> NHD
            assert torch.equal(packed[l * stride:(l + 1) * stride], want.view(-1)), ("pack", l)
            exp = torch.full_like(dst[l][0], 0xA5).view(nblk, 2, heads, ntpb, row)
            exp.index_copy_(0, d_ids, picked)
            assert torch.equal(dst[l][0].view(nblk, 2, heads, ntpb, row), exp), ("unpack", l)
            del want, exp, picked
        del src, dst, sc, dc, packed
        torch.cuda.empty_cache()


def _run_runs(w, seed):
    """The same check for a TP-remapping batch through a run plan (the per-token arithmetic
    evaluated in the kernel): the oracle's per-token lists, unmerged, drive torch's gather and
    scatter."""
    plan, runs = pipeline.build_plan_runs(w, 0)
    o_lists = _oracle_lists(w)
    assert plan.num_strided_chunks > 0
    src, dst = _caches(w, seed)
    sc = kvt_amd.Cache(0, src, w.capacities("src"))
    dc = kvt_amd.Cache(0, dst, w.capacities("dst"))
    stride = plan.layer_bytes
    packed = torch.zeros(w.n_layers * stride, dtype=torch.uint8, device="cuda")
    plan.pack(sc, 0, w.n_layers, packed, stride)
    plan.unpack(dc, 0, w.n_layers, packed, stride)
    torch.cuda.synchronize()
    for t in range(w.n_tensors):
        ranges = o_lists[t]
        s_idx = torch.from_numpy(_unit_index(ranges[:, 0], ranges[:, 2])).cuda()
        d_idx = torch.from_numpy(_unit_index(ranges[:, 1], ranges[:, 2])).cuda()
        assert len(torch.unique(d_idx)) == len(d_idx)
        nb = int(ranges[:, 2].sum())
        assert plan.tensor_bytes(t) == nb
        off = plan.tensor_offset(t)
        for l in range(w.n_layers):
            blob = packed[l * stride + off: l * stride + off + nb].view(-1, 16)
            assert _gathered_equals(src[l][t].view(-1, 16), s_idx, blob), ("pack", l, t)
            exp = torch.full_like(dst[l][t], 0xA5).view(-1, 16)
            _scatter(exp, d_idx, blob)
            assert torch.equal(dst[l][t].view(-1, 16), exp), ("unpack", l, t)
            del exp
    return plan, o_lists


def test_tp2_to_tp1_batch_full_size_through_a_run_plan():
    """Config 2's batch sent from TP2 to TP1: 623 786 per-token ranges of 1 KiB per layer,
    32 layers, 19 GiB payload."""
    w = workloads.tp_split("flash", 2, 1, 0, n_layers=32, src_pool=16384, dst_pool=24576,
                           n_req=64, min_tok=1024, max_tok=8192)
    plan, o_lists = _run_runs(w, 7)
    assert len(o_lists[0]) > 600000 and plan.num_chunks < 50000


def test_hybrid_tp2_to_tp1_full_size_through_a_run_plan():
    """The hybrid model between a TP2 prefill and a TP1 decode instance at the size of the
    benchmark (128 requests x 4096 tokens, 12 attention layers with their GDN states)."""
    w = workloads.qwen3next_tp_split(2, 1, 0, n_layers=12, pool=1024, n_req=128)
    _run_runs(w, 8)
