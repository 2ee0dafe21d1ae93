"""The CU-share limit of copy launches (kvt_set_copy_cu_usage, the reference's
BLLM_KVTRANS_KERNEL_COPY_SM_USAGE, kvtransfer/src/envcfg.cpp:311-326 and
copy_kernels.cpp:327-335): with a share below 1 every kernel runs as a bounded
number of persistent workgroups striding over the same work, so every result
must be bit for bit what the unlimited launch gives. The parity tests of the
other GPU test files are run again under two limits: half the device, and the
smallest grid the library will use (8 workgroups on a 256-CU part at 0.004).
Needs a real MI355X."""
import ctypes as C
import math

import numpy as np
import pytest

import checkers
import kvt_amd
import test_gpu_pack as tp
import test_gpu_runs as tr
from kvt_amd import pipeline, workloads

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(params=[0.5, 0.004], ids=["half", "eight-workgroups"])
def limited(request):
    kvt_amd.set_copy_cu_usage(0, request.param)
    try:
        yield request.param
    finally:
        kvt_amd.set_copy_cu_usage(0, 1.0)


def test_setting_and_reading_the_share():
    lib = kvt_amd.lib()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    try:
        assert kvt_amd.get_copy_cu_usage(0) == (1.0, 0)
        kvt_amd.set_copy_cu_usage(0, 0.25)
        usage, limit = kvt_amd.get_copy_cu_usage(0)
        assert usage == 0.25 and limit == (int(0.25 * cus * 8) & ~7) and limit % 8 == 0
        kvt_amd.set_copy_cu_usage(0, 1 / 3)
        assert kvt_amd.get_copy_cu_usage(0) == (1 / 3, int(cus * 8 / 3) & ~7)
        kvt_amd.set_copy_cu_usage(0, 1e-6)
        assert kvt_amd.get_copy_cu_usage(0)[1] == 8
        kvt_amd.set_copy_cu_usage(0, 1.0)
        assert kvt_amd.get_copy_cu_usage(0) == (1.0, 0)
        for bad in (0.0, -0.5, 1.5, math.nan, math.inf):
            assert lib.kvt_set_copy_cu_usage(0, bad) != 0, bad
            assert b"usage" in lib.kvt_last_error()
        assert lib.kvt_set_copy_cu_usage(99, 0.5) != 0
        assert lib.kvt_get_copy_cu_usage(99, None, None) != 0
        assert lib.kvt_get_copy_cu_usage(0, None, None) == 0
        assert kvt_amd.get_copy_cu_usage(0) == (1.0, 0)      # refused values change nothing
    finally:
        assert lib.kvt_set_copy_cu_usage(0, C.c_double(1.0)) == 0


def test_plain_plans_under_a_limit(limited):
    tp.test_config2_shape_reduced_pool(0)
    tp.test_config2_shape_reduced_pool(65536)
    tp.test_config4_mla_and_indexer_two_tensors()
    tp.test_config5_reference_layout_uniform_pages_shared_by_attention_and_gdn()
    tp.test_chunked_prefill_steps_and_ragged_tail()
    tp.test_arbitrary_ranges_including_misaligned()


def test_short_plans_in_kernel_arguments_under_a_limit(limited):
    for n in (1, 63, 64, 65):
        tp.test_short_plans_travel_in_the_kernel_arguments(n)


def test_transposing_plans_under_a_limit(limited):
    tp.test_config3_transposing_pack_hnd_to_nhd()
    tp.test_transposing_pack_other_geometries(3, 5, 48)


def test_strided_and_converting_plans_under_a_limit(limited):
    tr.test_tp_split_batches_through_a_run_plan("flash", 2, 1, 1, True, 0)
    tr.test_tp_split_batches_through_a_run_plan("ragged", 1, 4, 0, True, 4096)
    tr.test_hybrid_model_between_tp2_prefill_and_tp1_decode(2, 1, 1)
    tr.test_strided_plan_with_word_aligned_and_misaligned_blob_positions()
    tr.test_converting_run_plan_bf16_sender_fp8_receiver("flash", 2, 1, 1, 0, "raw")
    tr.test_converting_plan_of_plain_unaligned_ranges_takes_the_element_path()


def test_reference_shaped_entry_points_under_a_limit(limited):
    tp.test_launch_copy_direct_gather_and_scatter(5, 200000)
    tp.test_launch_copy_direct_gather_and_scatter(5000, 700)
    tp.test_copy_handle_data_with_kernel_pinned_host_buffer(7)
    tp.test_copy_handle_data_kernel_direct(False)
    tp.test_bf16_to_fp8_all_bit_patterns_and_converting_gather()


def test_sessions_and_graphs_under_a_limit(limited):
    tp.test_per_layer_session_on_side_stream()
    tp.test_session_inside_hip_graph_replays()
    tp.test_stager_save_load_round_trip_overlapped_with_packing()


@pytest.mark.parametrize("usage", [0.25, 0.1, 0.004], ids=["quarter", "tenth", "eight-workgroups"])
@pytest.mark.parametrize("chunk", [0, 4096, 8192, 16384, 32768, 65536, 524288])
def test_pipelined_kernels_of_strided_transposing_and_converting_plans(usage, chunk):
    """Below half the device, strided, transposing and converting tables are moved by
    persistent workgroups that take whole table entries (in parts of 16 or 32 KiB; entries of
    4 or 8 KiB: a wavefront each) through buffer descriptors with 32-bit offsets computed per lane. Batches large enough for a full
    grid of them, every entry size, both directions, against the oracle."""
    kvt_amd.set_copy_cu_usage(0, usage)
    try:
        for layout, p_tp, d_tp, rank in (("flash", 2, 1, 1), ("ragged", 4, 2, 3), ("ragged", 1, 4, 0),
                                         ("hnd", 2, 1, 1), ("flash", 8, 1, 3), ("ragged", 2, 8, 1)):
            w = workloads.tp_split(layout, p_tp, d_tp, rank, n_layers=4, src_pool=500, dst_pool=600,
                                   n_req=6, min_tok=200, max_tok=1400)
            plan, runs = pipeline.build_plan_runs(w, 0, chunk)
            tr._check(w, plan, tr._oracle_ranges(w), 91, None)
        for layout, p_tp, d_tp, rank in (("flash", 2, 1, 1), ("ragged", 8, 2, 5)):
            w = workloads.tp_split(layout, p_tp, d_tp, rank, n_layers=4, src_pool=500, dst_pool=600,
                                   n_req=6, min_tok=200, max_tok=1400, fp8_dst=True)
            tr._check_converting(w, chunk, "raw")
        if chunk in (0, 32768, 65536):   # a chunk holds whole token rows of the transform
            w = workloads.llama70b_flashinfer(n_layers=4, pool=400, n_req=4, tokens=1500)
            plan, lists = pipeline.build_plan(w, 0, chunk)
            tp._transposing(w, plan=plan, lists=lists)
        if chunk in (0, 4096, 8192):     # one rank of TP4 / TP8: half pages of 8 / 4 KiB
            for heads in (2, 1):
                w = workloads.llama70b_flashinfer(n_layers=4, pool=1200, n_req=6, tokens=3000, heads=heads)
                plan, lists = pipeline.build_plan(w, 0, chunk)
                tp._transposing(w, plan=plan, lists=lists)
    finally:
        kvt_amd.set_copy_cu_usage(0, 1.0)


@pytest.mark.parametrize("usage", [0.5, 0.1, 0.004], ids=["half", "tenth", "eight-workgroups"])
@pytest.mark.parametrize("chunk", [4096, 8192])
def test_wavefront_per_entry_kernel_of_plain_tables_with_small_entries(usage, chunk):
    """A limited launch of a plain, 16-byte aligned table cut into entries of 4 or 8 KiB gives
    every wavefront entries of its own. Seeded batches of arbitrary 16-byte aligned ranges: 1-3
    tensors, 1-5 layers, lengths from 16 bytes to 70 000 (entries shorter than a wavefront's
    reach, tables that do not fill the last trip), shuffled, enough of them for a full grid at
    half the device (with counters) and at a tenth (without), against the oracle."""
    kvt_amd.set_copy_cu_usage(0, usage)
    try:
        for seed in range(6):
            rng = np.random.default_rng(77_000 + seed)
            n_t, n_layers = int(rng.integers(1, 4)), int(rng.integers(1, 6))
            caps_s = [int(rng.integers(1 << 22, 1 << 23)) // 16 * 16 for _ in range(n_t)]
            caps_d = [int(rng.integers(1 << 22, 1 << 23)) // 16 * 16 for _ in range(n_t)]
            lists, all_runs = kvt_amd.BlockLists(), []
            for t in range(n_t):
                runs, d = [], 0
                while len(runs) < 400:
                    ln = int(rng.choice([16, 48, 1024, 4096, 4112, 5008, 8192, 12288, 36864, 69984]))
                    gap = int(rng.integers(0, 4)) * 16
                    if d + gap + ln > caps_d[t]:
                        break
                    s_off = int(rng.integers(0, (caps_s[t] - ln) // 16 + 1)) * 16
                    runs.append((s_off, d + gap, ln))
                    d += gap + ln
                runs = [runs[i] for i in rng.permutation(len(runs))]
                lists.append(t, runs)
                all_runs.append(np.asarray(runs, np.uint64))
            plan = kvt_amd.Plan(0, lists, caps_s, caps_d, chunk_bytes=chunk)
            src = [[tp._dev_bytes(c, seed * 64 + l * 8 + t, "u8") for t, c in enumerate(caps_s)]
                   for l in range(n_layers)]
            dst = [[torch.full((c,), 0xA5, device="cuda", dtype=torch.uint8) for c in caps_d]
                   for _ in range(n_layers)]
            sc, dc = kvt_amd.Cache(0, src, caps_s), kvt_amd.Cache(0, dst, caps_d)
            stride = plan.layer_bytes + 256
            packed = torch.zeros(n_layers * stride, dtype=torch.uint8, device="cuda")
            plan.pack(sc, 0, n_layers, packed, stride)
            plan.unpack(dc, 0, n_layers, packed, stride)
            torch.cuda.synchronize()
            ph = tp._host(packed)
            for l in range(n_layers):
                for t in range(n_t):
                    blob = checkers.oracle_pack(tp._host(src[l][t]), all_runs[t])
                    off = l * stride + plan.tensor_offset(t)
                    assert np.array_equal(ph[off:off + len(blob)], blob), (seed, l, t)
                    exp = np.full(caps_d[t], 0xA5, dtype=np.uint8)
                    checkers.oracle_unpack(exp, all_runs[t], blob)
                    assert np.array_equal(tp._host(dst[l][t]), exp), (seed, l, t)
            plan.close()
    finally:
        kvt_amd.set_copy_cu_usage(0, 1.0)


@pytest.mark.parametrize("usage", [0.1, 0.004], ids=["tenth", "eight-workgroups"])
@pytest.mark.parametrize("chunk", [4096, 8192, 16384, 32768])
def test_short_tables_in_kernel_arguments_entry_by_entry_under_a_limit(usage, chunk):
    """A table of at most 64 entries travels in the kernel arguments; under a limit, with more
    (entry, layer) pairs than workgroups, the persistent kernels read it from there. Every entry
    size, entries shorter than the size, two tensors, 40 layers, against the oracle."""
    kvt_amd.set_copy_cu_usage(0, usage)
    try:
        for seed, n_ranges in enumerate((3, 32)):
            rng = np.random.default_rng(88_000 + seed)
            caps = [1 << 21, 1 << 21]
            n_layers = 40
            lists, all_runs = kvt_amd.BlockLists(), []
            for t in range(2):
                runs, d = [], 0
                for _ in range(n_ranges):
                    ln = int(rng.choice([16, 2048, chunk - 16, chunk]))
                    s_off = int(rng.integers(0, (caps[t] - ln) // 16)) * 16
                    runs.append((s_off, d, ln))
                    d += ln + int(rng.integers(0, 3)) * 16
                runs = [runs[i] for i in rng.permutation(len(runs))]
                lists.append(t, runs)
                all_runs.append(np.asarray(runs, np.uint64))
            plan = kvt_amd.Plan(0, lists, caps, caps, chunk_bytes=chunk)
            src = [[tp._dev_bytes(c, seed * 640 + l * 8 + t, "u8") for t, c in enumerate(caps)]
                   for l in range(n_layers)]
            dst = [[torch.full((c,), 0x5A, device="cuda", dtype=torch.uint8) for c in caps]
                   for _ in range(n_layers)]
            sc, dc = kvt_amd.Cache(0, src, caps), kvt_amd.Cache(0, dst, caps)
            stride = plan.layer_bytes
            packed = torch.zeros(n_layers * stride, dtype=torch.uint8, device="cuda")
            plan.pack(sc, 0, n_layers, packed, stride)
            plan.unpack(dc, 0, n_layers, packed, stride)
            torch.cuda.synchronize()
            ph = tp._host(packed)
            for l in range(n_layers):
                for t in range(2):
                    blob = checkers.oracle_pack(tp._host(src[l][t]), all_runs[t])
                    off = l * stride + plan.tensor_offset(t)
                    assert np.array_equal(ph[off:off + len(blob)], blob), (seed, l, t)
                    exp = np.full(caps[t], 0x5A, dtype=np.uint8)
                    checkers.oracle_unpack(exp, all_runs[t], blob)
                    assert np.array_equal(tp._host(dst[l][t]), exp), (seed, l, t)
            plan.close()
    finally:
        kvt_amd.set_copy_cu_usage(0, 1.0)


@pytest.mark.parametrize("usage", [0.25, 0.004], ids=["quarter", "eight-workgroups"])
@pytest.mark.parametrize("block", [4096, 32768])
def test_converting_plan_of_plain_aligned_ranges_under_a_limit(usage, block):
    """Same TP on both sides, bf16 sender and fp8 receiver: plain ranges of whole blocks. The
    pack converts through the persistent converting kernels (entries of 4096 elements: a
    wavefront each), the unpack moves plain fp8 bytes through the persistent copy kernels."""
    rng = np.random.default_rng(block)
    n_blocks, n_layers, pool = 700, 3, 1000
    src_ids = rng.permutation(pool)[:n_blocks]
    dst_ids = rng.permutation(pool)[:n_blocks]
    elems = block // 2                                         # a block holds bf16
    ranges = np.stack([src_ids * block, dst_ids * elems, np.full(n_blocks, elems)], axis=1).astype(np.uint64)
    lists = kvt_amd.BlockLists()
    lists.append(0, ranges)
    cap_s, cap_d = pool * block, pool * elems
    plan = kvt_amd.Plan(0, kvt_amd.RunLists.compress(lists), [cap_s], [cap_d], bf16_to_fp8=True)
    src = [[tp._dev_bytes(cap_s, 30 + l, "raw")] for l in range(n_layers)]
    dst = [[torch.full((cap_d,), 0xA5, dtype=torch.uint8, device="cuda")] for _ in range(n_layers)]
    stride = plan.layer_bytes
    packed = torch.zeros(n_layers * stride, dtype=torch.uint8, device="cuda")
    kvt_amd.set_copy_cu_usage(0, usage)
    try:
        plan.pack(kvt_amd.Cache(0, src, [cap_s]), 0, n_layers, packed, stride)
        plan.unpack(kvt_amd.Cache(0, dst, [cap_d]), 0, n_layers, packed, stride)
        torch.cuda.synchronize()
    finally:
        kvt_amd.set_copy_cu_usage(0, 1.0)
    for l in range(n_layers):
        blob = tr._oracle_pack_fp8(tp._host(src[l][0]), ranges)
        assert np.array_equal(tp._host(packed)[l * stride:l * stride + len(blob)], blob), l
        exp = np.full(cap_d, 0xA5, dtype=np.uint8)
        checkers.oracle_unpack(exp, ranges, blob)
        assert np.array_equal(tp._host(dst[l][0]), exp), l


def test_more_limited_launches_in_flight_than_ticket_blocks():
    """A limited launch of the pipelined kernels borrows a block of counters until it has run.
    At an eighth of the device such a launch asks for one (a workgroup per CU). Thousands of
    launches queued behind a kernel that holds the stream back outnumber the blocks: those that
    find none run without (every workgroup a fixed share), and once the queue has drained the
    blocks are lent again, each left zeroed by the launch that had it. Every result is the
    oracle's, and the library's counters show that both paths were taken."""
    w = workloads.llama8b_single(n_layers=4, pool=256, tokens=2048)
    plan, lists = pipeline.build_plan(w, 0)
    assert plan.num_chunks > 64                      # a resident table, not kernel arguments
    o_lists = tp._oracle_lists(w)
    src_layers = tp._make_caches(w, "src", 17)
    sc = kvt_amd.Cache(0, src_layers, w.capacities("src"))
    stride = plan.layer_bytes
    outs = [torch.zeros(w.n_layers * stride, dtype=torch.uint8, device="cuda") for _ in range(3)]
    blobs = [checkers.oracle_pack(tp._host(src_layers[l][0]), o_lists[0]) for l in range(w.n_layers)]

    def check():
        for l in range(w.n_layers):
            for out in outs:
                assert np.array_equal(tp._host(out)[l * stride:l * stride + len(blobs[l])], blobs[l]), l

    kvt_amd.set_copy_cu_usage(0, 0.125)
    try:
        stream = checkers.side_stream()
        got0, none0 = kvt_amd.copy_ticket_stats(0)[:2]
        with torch.cuda.stream(stream):
            torch.cuda._sleep(400_000_000)           # some tenths of a second: the launches pile up
        for i in range(3000):
            plan.pack(sc, 0, w.n_layers, outs[i % 3], stride, stream.cuda_stream)
        got1, none1 = kvt_amd.copy_ticket_stats(0)[:2]
        stream.synchronize()
        check()
        assert got1 - got0 > 0 and none1 - none0 > 0, (got0, none0, got1, none1)
        assert (got1 - got0) + (none1 - none0) == 3000
        # every block has been through a launch: the next ones reuse them
        for out in outs:
            out.zero_()
        torch.cuda.synchronize()
        for i in range(1500):
            plan.pack(sc, 0, w.n_layers, outs[i % 3], stride, stream.cuda_stream)
            if i % 100 == 99:
                stream.synchronize()
        stream.synchronize()
        got2, none2 = kvt_amd.copy_ticket_stats(0)[:2]
        assert got2 - got1 >= 1400, (got1, none1, got2, none2)
        check()
    finally:
        kvt_amd.set_copy_cu_usage(0, 1.0)


@pytest.mark.parametrize("usage", [0.25, 0.004], ids=["quarter", "eight-workgroups"])
def test_limited_launches_of_every_pipelined_kernel_inside_a_graph(usage):
    """A limited launch recorded into a hipGraph keeps a block of counters of its own for every
    replay. Plain, strided, converting and transposing plans (entries a workgroup takes and
    entries a wavefront takes), pack and unpack in one graph,
    replayed with fresh cache contents each time."""
    kvt_amd.set_copy_cu_usage(0, usage)
    try:
        cases = []
        w = workloads.llama8b_batch(n_layers=3, src_pool=700, dst_pool=900, n_req=6, min_tok=300, max_tok=1500)
        cases.append((w, pipeline.build_plan(w, 0)[0]))
        w = workloads.deepseek_mla(n_layers=3, pool=700, n_req=4, tokens=8192)   # 4 KiB entries
        cases.append((w, pipeline.build_plan(w, 0)[0]))
        w = workloads.tp_split("flash", 2, 1, 1, n_layers=3, src_pool=500, dst_pool=600, n_req=6,
                               min_tok=200, max_tok=1400)
        cases.append((w, pipeline.build_plan_runs(w, 0)[0]))
        w = workloads.tp_split("flash", 2, 1, 1, n_layers=3, src_pool=500, dst_pool=600, n_req=6,
                               min_tok=200, max_tok=1400, fp8_dst=True)
        cases.append((w, pipeline.build_plan_runs(w, 0)[0]))
        w = workloads.llama70b_flashinfer(n_layers=3, pool=400, n_req=4, tokens=1500)
        cases.append((w, pipeline.build_plan(w, 0)[0]))
        # entries of 4 and 8 KiB (one or two KV heads per rank): a wavefront per entry
        w = workloads.tp_split("flash", 8, 1, 3, n_layers=3, src_pool=900, dst_pool=1000, n_req=6,
                               min_tok=400, max_tok=2400)
        cases.append((w, pipeline.build_plan_runs(w, 0)[0]))
        w = workloads.tp_split("flash", 8, 1, 3, n_layers=3, src_pool=900, dst_pool=1000, n_req=6,
                               min_tok=400, max_tok=2400, fp8_dst=True)
        cases.append((w, pipeline.build_plan_runs(w, 0)[0]))
        w = workloads.llama70b_flashinfer(n_layers=3, pool=1200, n_req=6, tokens=3000, heads=2)
        cases.append((w, pipeline.build_plan(w, 0)[0]))
        for w, plan in cases:
            plan.ready()
            src = tp._make_caches(w, "src", 5, dtype="raw" if w.notes.get("fp8") else None)
            sc = kvt_amd.Cache(0, src, w.capacities("src"))
            stride = plan.layer_bytes
            eager = torch.zeros(w.n_layers * stride, dtype=torch.uint8, device="cuda")
            out = torch.zeros_like(eager)
            dst_e = tp._make_caches(w, "dst", 6, fill=False)
            dst_g = tp._make_caches(w, "dst", 6, fill=False)
            de, dg = (kvt_amd.Cache(0, d, w.capacities("dst")) for d in (dst_e, dst_g))
            graph = torch.cuda.CUDAGraph()
            cs = checkers.side_stream()
            with torch.cuda.graph(graph, stream=cs):
                plan.pack(sc, 0, w.n_layers, out, stride, cs.cuda_stream)
                plan.unpack(dg, 0, w.n_layers, out, stride, cs.cuda_stream)
            for rep in range(3):
                for l in range(w.n_layers):
                    for t in range(w.n_tensors):
                        src[l][t].copy_(torch.roll(src[l][t], 4096 * (rep + 1)))
                torch.cuda.synchronize()
                graph.replay()
                kvt_amd.set_copy_cu_usage(0, 1.0)       # the unlimited launches as the reference
                plan.pack(sc, 0, w.n_layers, eager, stride)
                plan.unpack(de, 0, w.n_layers, eager, stride)
                kvt_amd.set_copy_cu_usage(0, usage)
                torch.cuda.synchronize()
                assert torch.equal(out, eager), (w.name, rep)
                for l in range(w.n_layers):
                    for t in range(w.n_tensors):
                        assert torch.equal(dst_g[l][t], dst_e[l][t]), (w.name, rep, l, t)
    finally:
        kvt_amd.set_copy_cu_usage(0, 1.0)


def test_limited_launches_of_one_plan_from_several_threads_at_once():
    """Launches that may run at the same time never share a block of counters: four threads,
    each on a stream of its own, pack the same plan under a limit into their own buffers."""
    import threading
    w = workloads.llama8b_batch(n_layers=2, src_pool=700, dst_pool=900, n_req=6, min_tok=300, max_tok=1500)
    plan, lists = pipeline.build_plan(w, 0)
    plan.ready()
    src_layers = tp._make_caches(w, "src", 23)
    sc = kvt_amd.Cache(0, src_layers, w.capacities("src"))
    stride = plan.layer_bytes
    outs = [torch.zeros(w.n_layers * stride, dtype=torch.uint8, device="cuda") for _ in range(4)]
    errors = []

    def worker(i):
        try:
            st = checkers.side_stream()
            for _ in range(60):
                plan.pack(sc, 0, w.n_layers, outs[i], stride, st.cuda_stream)
            st.synchronize()
        except Exception as e:          # noqa: BLE001 - handed to the main thread
            errors.append(e)

    kvt_amd.set_copy_cu_usage(0, 0.25)
    try:
        threads = [threading.Thread(target=worker, args=(i,)) for i in range(4)]
        for t in threads:
            t.start()
        for t in threads:
            t.join(120)
    finally:
        kvt_amd.set_copy_cu_usage(0, 1.0)
    assert not errors, errors
    o_lists = tp._oracle_lists(w)
    for l in range(w.n_layers):
        blob = checkers.oracle_pack(tp._host(src_layers[l][0]), o_lists[0])
        for out in outs:
            assert np.array_equal(tp._host(out)[l * stride:l * stride + len(blob)], blob), l
