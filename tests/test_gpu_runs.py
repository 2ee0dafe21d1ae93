"""GPU parity of plans built from strided runs (the per-token / per-head offset
arithmetic of the TP-remapping parsers evaluated inside the copy kernel) against
the CPU oracle's pack / unpack of the oracle's own per-token range lists.
Bit-exact. Needs a real MI355X."""
import numpy as np
import pytest

import cases
import checkers
import kvt_amd
from kvt_amd import pipeline, workloads
from test_gpu_pack import _dev_bytes, _host, _make_caches

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _oracle_ranges(w):
    src, dst = w.worker_infos()
    rc, valid, tps, tpr, pid, kind = checkers.oracle_select(w.cache_shape, src, dst)
    assert rc == 0 and kind != 0          # never merged
    rc, outs = checkers.oracle_parse(pid, src, dst, valid, tps, tpr, w.task_bufs())
    assert rc == 0
    return outs


def _check(w, plan, o_lists, seed, expect_strided):
    if expect_strided is not None:
        assert (plan.num_strided_chunks > 0) == expect_strided
    src_layers = _make_caches(w, "src", seed)
    dst_layers = _make_caches(w, "dst", seed + 1, fill=False)
    sc = kvt_amd.Cache(0, src_layers, w.capacities("src"))
    dc = kvt_amd.Cache(0, dst_layers, w.capacities("dst"))
    stride = plan.layer_bytes
    packed = torch.zeros(w.n_layers * stride, dtype=torch.uint8, device="cuda")
    plan.pack(sc, 0, w.n_layers, packed, stride)
    torch.cuda.synchronize()
    packed_h = _host(packed)
    for l in range(w.n_layers):
        for t in range(w.n_tensors):
            blob = checkers.oracle_pack(_host(src_layers[l][t]), o_lists[t])
            off = l * stride + plan.tensor_offset(t)
            assert plan.tensor_bytes(t) == len(blob)
            assert np.array_equal(packed_h[off:off + len(blob)], blob), (l, t)
    plan.unpack(dc, 0, w.n_layers, packed, stride)
    torch.cuda.synchronize()
    for l in range(w.n_layers):
        for t in range(w.n_tensors):
            exp = np.full(w.capacities("dst")[t], 0xA5, dtype=np.uint8)
            off = l * stride + plan.tensor_offset(t)
            checkers.oracle_unpack(exp, o_lists[t], packed_h[off:off + plan.tensor_bytes(t)])
            assert np.array_equal(_host(dst_layers[l][t]), exp), (l, t)


SPLITS = [("flash", 2, 1, 1, True), ("flash", 4, 1, 2, True), ("ragged", 1, 2, 1, True),
          ("ragged", 4, 2, 3, True), ("ragged", 1, 4, 0, True), ("hnd", 2, 1, 1, None)]   # hnd: whole-segment head rows (plain), short tails strided


@pytest.mark.parametrize("layout,p_tp,d_tp,rank,strided", SPLITS)
@pytest.mark.parametrize("chunk", [0, 4096, 65536])
def test_tp_split_batches_through_a_run_plan(layout, p_tp, d_tp, rank, strided, chunk):
    w = workloads.tp_split(layout, p_tp, d_tp, rank, n_layers=3, src_pool=300, dst_pool=400,
                           n_req=5, min_tok=30, max_tok=900)
    plan, runs = pipeline.build_plan_runs(w, 0, chunk)
    o_lists = _oracle_ranges(w)
    assert np.array_equal(runs.expand().tensor(0), o_lists[0])
    assert len(runs.tensor(0)) < len(o_lists[0])
    _check(w, plan, o_lists, 51, strided)


@pytest.mark.parametrize("p_tp,d_tp,rank", [(2, 1, 0), (2, 1, 1)])
def test_hybrid_model_between_tp2_prefill_and_tp1_decode(p_tp, d_tp, rank):
    """Attention pages split per token inside kernel blocks, GDN conv rows split per channel
    group, one SSM range, and the zero fill of the receiver's last page, all in one batch;
    destination tables are disjoint, so the scatter is checked as well."""
    w = workloads.qwen3next_tp_split(p_tp, d_tp, rank, n_layers=2, pool=64, n_req=6, tokens=1500)
    plan, runs = pipeline.build_plan_runs(w, 0)
    o_lists = _oracle_ranges(w)
    assert np.array_equal(runs.expand().tensor(0), o_lists[0])
    lens = o_lists[0][:, 2]
    assert lens.min() <= 512 and lens.max() >= 1 << 20          # token rows up to SSM states
    _check(w, plan, o_lists, 71, True)


def test_receiver_compresses_plain_ranges_then_unpacks_strided():
    w = workloads.tp_split("flash", 2, 1, 0, n_layers=2, src_pool=200, dst_pool=300, n_req=4,
                           min_tok=100, max_tok=700)
    o_lists = _oracle_ranges(w)
    lists = kvt_amd.BlockLists()
    lists.append(0, o_lists[0])                      # as taken off a layer message
    runs = kvt_amd.RunLists.compress(lists)
    plan = kvt_amd.Plan(0, runs, w.capacities("src"), w.capacities("dst"))
    _check(w, plan, o_lists, 61, True)
    plain = kvt_amd.Plan(0, lists, w.capacities("src"), w.capacities("dst"))
    assert plan.layer_bytes == plain.layer_bytes and plan.num_chunks * 3 < plain.num_chunks


PER_TOKEN = ["RAGGED_PGTD", "RAGGED_PLTD", "FLASH_PGTD", "DPSK_PGTD", "DPSK_PLTD",
             "FLASHINFER_PGTD", "HYBRID_PGTD", "HYBRID_PLTD", "HYBRID_FI_PGTD", "HYBRID_FI_PLTD",
             "KDA_PGTD", "KIMI_K3_PLTD", "TURBOQUANT_PGTD"]


@pytest.mark.parametrize("parser", PER_TOKEN)
def test_pack_of_random_cases_of_every_remapping_parser(parser):
    """Gather only: the random cases may repeat destination blocks."""
    done = 0
    for seed in range(900, 1100):
        case = cases.gen_case(parser, seed)
        pid, src, dst, valid, tps, tpr, tasks = cases.materialise(case)
        rc, outs = checkers.oracle_parse(pid, src, dst, valid, tps, tpr, tasks)
        if rc != 0 or not any(len(o) for o in outs) or any(len(o) == 0 for o in outs):
            continue
        parser_h = kvt_amd.Parser(pid, src, dst, valid, tps, tpr)
        runs = kvt_amd.RunLists()
        for t in tasks:
            assert parser_h.parse_runs(t.struct, runs) == 0
        n_t = runs.num_tensors()
        s_cap = [int(src.block_sizes[t]) * int(src.layer_num_blocks) for t in range(n_t)]
        d_cap = [int(dst.block_sizes[t]) * int(dst.layer_num_blocks) for t in range(n_t)]
        plan = kvt_amd.Plan(0, runs, s_cap, d_cap)
        layers = [[_dev_bytes((c + 3) // 4 * 4, seed * 10 + t, "u8") for t, c in enumerate(s_cap)]]
        cache = kvt_amd.Cache(0, layers, s_cap)
        packed = torch.zeros(max(plan.layer_bytes, 16), dtype=torch.uint8, device="cuda")
        plan.pack(cache, 0, 1, packed, plan.layer_bytes)
        torch.cuda.synchronize()
        packed_h = _host(packed)
        for t in range(n_t):
            blob = checkers.oracle_pack(_host(layers[0][t]), outs[t])
            off = plan.tensor_offset(t)
            assert np.array_equal(packed_h[off:off + len(blob)], blob), (case["name"], t)
        done += 1
        if done == 12:
            break
    assert done >= 4


def test_strided_plan_with_word_aligned_and_misaligned_blob_positions():
    """16-byte aligned positions: one vector per lane; 4-byte aligned ones (a blob inside a
    layer message): word-wise path, same bytes; anything else is refused."""
    w = workloads.tp_split("flash", 2, 1, 0, n_layers=2, src_pool=64, dst_pool=64, n_req=2,
                           min_tok=100, max_tok=300)
    plan, _ = pipeline.build_plan_runs(w, 0)
    assert plan.num_strided_chunks > 0
    o_runs = _oracle_ranges(w)[0]
    layers = _make_caches(w, "src", 5)
    sc = kvt_amd.Cache(0, layers, w.capacities("src"))
    for off, stride_pad in ((32, 0), (4, 0), (12, 4), (44, 8)):
        stride = plan.layer_bytes + 64 + stride_pad
        out = torch.zeros(w.n_layers * stride, dtype=torch.uint8, device="cuda")
        plan.pack_at(sc, 0, w.n_layers, out, stride, [off] + [0] * 7)
        dst_layers = _make_caches(w, "dst", 6, fill=False)
        dc = kvt_amd.Cache(0, dst_layers, w.capacities("dst"))
        plan.unpack_at(dc, 0, w.n_layers, out, stride, [off] + [0] * 7)
        torch.cuda.synchronize()
        out_h = _host(out)
        for l in range(w.n_layers):
            blob = checkers.oracle_pack(_host(layers[l][0]), o_runs)
            assert np.array_equal(out_h[l * stride + off: l * stride + off + len(blob)], blob), (off, l)
            exp = np.full(w.capacities("dst")[0], 0xA5, dtype=np.uint8)
            checkers.oracle_unpack(exp, o_runs, blob)
            assert np.array_equal(_host(dst_layers[l][0]), exp), (off, l)
    out = torch.zeros(plan.layer_bytes + 64, dtype=torch.uint8, device="cuda")
    with pytest.raises(kvt_amd.KvtError):
        plan.pack_at(sc, 0, 1, out, 0, [1] + [0] * 7)
    with pytest.raises(kvt_amd.KvtError):
        plan.pack_at(sc, 0, 1, out.data_ptr() + 2, 0, [0] * 8)


@pytest.mark.parametrize("seed", range(8))
def test_random_synthetic_runs_on_the_gpu(seed):
    """Runs no parser would emit (odd lengths, zero source strides, three levels, more record
    shapes than the kernel takes): gather and scatter against the oracle on the expanded list."""
    cap = 1 << 22
    runs = cases.gen_synthetic_runs(seed, cap, kvt_amd.binding.RUN_DTYPE)
    R = kvt_amd.RunLists()
    R.append(0, runs)
    expect = R.expand().tensor(0)
    plan = kvt_amd.Plan(0, R, [cap], [cap], chunk_bytes=[0, 4096, 65536][seed % 3])
    src = _dev_bytes(cap, 700 + seed, "u8")
    dst = torch.full((cap,), 0xA5, dtype=torch.uint8, device="cuda")
    sc, dc = kvt_amd.Cache(0, [[src]], [cap]), kvt_amd.Cache(0, [[dst]], [cap])
    packed = torch.zeros(max(plan.layer_bytes, 16), dtype=torch.uint8, device="cuda")
    plan.pack(sc, 0, 1, packed, plan.layer_bytes)
    plan.unpack(dc, 0, 1, packed, plan.layer_bytes)
    torch.cuda.synchronize()
    blob = checkers.oracle_pack(_host(src), expect)
    assert np.array_equal(_host(packed)[:len(blob)], blob)
    exp = np.full(cap, 0xA5, dtype=np.uint8)
    checkers.oracle_unpack(exp, expect, blob)
    assert np.array_equal(_host(dst), exp)


# ------------------------------------------- bf16 -> fp8 while gathering (resident plan)

def _oracle_pack_fp8(layer_h, ranges):
    """ranges: (src byte offset in the bf16 cache, dst, length in fp8 bytes = elements)"""
    r = np.ascontiguousarray(ranges, dtype=np.uint64)
    out = np.zeros(int(r[:, 2].sum()), dtype=np.uint8)
    checkers.oracle().kvto_pack_bf16_to_fp8(layer_h.ctypes.data, r.ctypes.data, len(r),
                                            out.ctypes.data)
    return out


# (ragged with p_tp = 2 d_tp is left out: an fp8 receiver then has the sender's token size, which
# the reference's dispatch takes for a replicated cache, tx_stub.cpp:451-590)
@pytest.mark.parametrize("layout,p_tp,d_tp,rank", [("flash", 2, 1, 1), ("flash", 4, 2, 3),
                                                   ("ragged", 8, 2, 5), ("ragged", 4, 1, 2)])
@pytest.mark.parametrize("chunk", [0, 4096, 65536])
@pytest.mark.parametrize("content", ["bf16", "raw"])
def test_converting_run_plan_bf16_sender_fp8_receiver(layout, p_tp, d_tp, rank, chunk, content):
    """The reference's BLLM_KVTRANS_BF162FP8_CONV mode: the P > D parsers emit fp8 lengths and
    the sender converts while it gathers. `raw` content makes every bf16 bit pattern
    (NaNs, infinities, denormals) likely."""
    w = workloads.tp_split(layout, p_tp, d_tp, rank, n_layers=2, src_pool=300, dst_pool=400,
                           n_req=4, min_tok=60, max_tok=900, fp8_dst=True)
    _check_converting(w, chunk, content)


def _check_converting(w, chunk, content):
    plan, runs = pipeline.build_plan_runs(w, 0, chunk)
    assert plan.num_strided_chunks > 0
    src_i, dst_i = w.worker_infos()
    rc, valid, tps, tpr, pid, kind = checkers.oracle_select(w.cache_shape, src_i, dst_i)
    assert rc == 0 and kind != 0
    rc, outs = checkers.oracle_parse(pid, src_i, dst_i, valid, tps, tpr, w.task_bufs(), fp8=True)
    assert rc == 0
    ranges = outs[0]
    assert np.array_equal(runs.expand().tensor(0), ranges)
    src_layers = _make_caches(w, "src", 91, dtype=content)
    dst_layers = _make_caches(w, "dst", 92, fill=False)
    sc = kvt_amd.Cache(0, src_layers, w.capacities("src"))
    dc = kvt_amd.Cache(0, dst_layers, w.capacities("dst"))
    stride = plan.layer_bytes
    assert plan.tensor_bytes(0) == int(ranges[:, 2].sum())        # fp8 bytes on the wire
    packed = torch.zeros(w.n_layers * stride, dtype=torch.uint8, device="cuda")
    plan.pack(sc, 0, w.n_layers, packed, stride)
    plan.unpack(dc, 0, w.n_layers, packed, stride)
    torch.cuda.synchronize()
    packed_h = _host(packed)
    for l in range(w.n_layers):
        blob = _oracle_pack_fp8(_host(src_layers[l][0]), ranges)
        assert np.array_equal(packed_h[l * stride:l * stride + len(blob)], blob), ("pack", l)
        exp = np.full(w.capacities("dst")[0], 0xA5, dtype=np.uint8)
        checkers.oracle_unpack(exp, ranges, blob)
        assert np.array_equal(_host(dst_layers[l][0]), exp), ("unpack", l)


def test_converting_plan_of_plain_unaligned_ranges_takes_the_element_path():
    rng = np.random.default_rng(5)
    cap_s, cap_d = 1 << 20, 1 << 19
    n = 24
    lens = rng.integers(1, 9000, size=n)                       # elements, any remainder mod 16
    s_off = np.sort(rng.choice(cap_s // 32768, size=n, replace=False)) * 32768 + 2 * rng.integers(0, 8, size=n)
    d_off = np.sort(rng.choice(cap_d // 16384, size=n, replace=False)) * 16384 + rng.integers(0, 16, size=n)
    ranges = np.stack([s_off, d_off, lens], axis=1).astype(np.uint64)
    lists = kvt_amd.BlockLists()
    lists.append(0, ranges)
    runs = kvt_amd.RunLists.compress(lists)
    plan = kvt_amd.Plan(0, runs, [cap_s], [cap_d], bf16_to_fp8=True)
    src = _dev_bytes(cap_s, 7, "raw")
    dst = torch.full((cap_d,), 0xA5, dtype=torch.uint8, device="cuda")
    packed = torch.zeros(max(plan.layer_bytes, 16), dtype=torch.uint8, device="cuda")
    plan.pack(kvt_amd.Cache(0, [[src]], [cap_s]), 0, 1, packed, plan.layer_bytes)
    plan.unpack(kvt_amd.Cache(0, [[dst]], [cap_d]), 0, 1, packed, plan.layer_bytes)
    torch.cuda.synchronize()
    blob = _oracle_pack_fp8(_host(src), ranges)
    assert np.array_equal(_host(packed)[:len(blob)], blob)
    exp = np.full(cap_d, 0xA5, dtype=np.uint8)
    checkers.oracle_unpack(exp, ranges, blob)
    assert np.array_equal(_host(dst), exp)
    # an odd source offset is not a bf16 element boundary
    bad = kvt_amd.BlockLists()
    bad.append(0, [(3, 0, 64)])
    with pytest.raises(kvt_amd.KvtError):
        kvt_amd.Plan(0, kvt_amd.RunLists.compress(bad), [cap_s], [cap_d], bf16_to_fp8=True)
    # the source side is checked at twice the length
    edge = kvt_amd.BlockLists()
    edge.append(0, [(cap_s - 64, 0, 64)])
    kvt_amd.Plan(0, kvt_amd.RunLists.compress(edge), [cap_s], [cap_d]).close()
    with pytest.raises(kvt_amd.KvtError):
        kvt_amd.Plan(0, kvt_amd.RunLists.compress(edge), [cap_s], [cap_d], bf16_to_fp8=True)
