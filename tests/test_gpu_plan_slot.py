"""Plan slots on the GPU (kvt_plan_slot_*): a plan at a fixed device address that takes a new
batch per fill, so that pack / unpack launches recorded ONCE into a hipGraph move a different
batch on every replay. The reference builds a new range list for every batch
(kvtransfer/src/tx_stub.cpp:158-263) and sends it layer by layer (:395-415); an engine whose
forward pass is a replayed graph needs the launches inside that graph to follow.
Every result is compared with the CPU oracle's pack / unpack of the oracle's own lists for THAT
batch. Needs a real MI355X."""
import threading
import time

import numpy as np
import pytest

import checkers
import kvt_amd
from kvt_amd import pipeline, workloads
from test_gpu_pack import _dev_bytes, _host, _make_caches, _oracle_lists

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _lists(w):
    src, dst = w.worker_infos()
    lists, _ = pipeline.parse_batch(w.cache_shape, src, dst, w.task_bufs())
    return lists


def _batch(seed, n_req, hi, n_layers=3, src_pool=512, dst_pool=768):
    return workloads.llama8b_batch(n_layers=n_layers, src_pool=src_pool, dst_pool=dst_pool, n_req=n_req,
                                   min_tok=20, max_tok=hi, seed=seed)


def _check_eager(slot, w, sc, dc, src_layers, dst_layers, packed, stride, stream, fill_with=None):
    """Fills the slot with w's batch, packs and unpacks every layer eagerly on `stream`, and
    compares with the oracle."""
    o_lists = _oracle_lists(w)
    lay = slot.fill(fill_with if fill_with is not None else _lists(w), stream.cuda_stream)
    for t in dst_layers:
        for x in t:
            x.fill_(0xA5)
    packed.zero_()
    torch.cuda.synchronize()
    slot.pack(sc, 0, w.n_layers, packed, stride, stream.cuda_stream)
    slot.unpack(dc, 0, w.n_layers, packed, stride, stream.cuda_stream)
    stream.synchronize()
    ph = _host(packed)
    for l in range(w.n_layers):
        for t in range(w.n_tensors):
            blob = checkers.oracle_pack(_host(src_layers[l][t]), o_lists[t])
            assert lay.tensor_bytes[t] == len(blob)
            off = l * stride + lay.tensor_offset[t]
            assert np.array_equal(ph[off:off + len(blob)], blob), (l, t)
            exp = np.full(w.capacities("dst")[t], 0xA5, dtype=np.uint8)
            checkers.oracle_unpack(exp, o_lists[t], blob)
            assert np.array_equal(_host(dst_layers[l][t]), exp), (l, t)
    return lay


@pytest.mark.parametrize("usage", [1.0, 0.25, 0.004], ids=["unlimited", "quarter", "eight-workgroups"])
@pytest.mark.parametrize("chunk", [0, 4096, 8192, 16384])
def test_eager_refills_of_a_plain_slot(chunk, usage):
    ws = [_batch(1, 6, 1500), _batch(2, 1, 100), _batch(3, 11, 700), _batch(4, 3, 2000)]
    w0 = ws[0]
    src_layers = _make_caches(w0, "src", 5)
    dst_layers = _make_caches(w0, "dst", 6, fill=False)
    sc = kvt_amd.Cache(0, src_layers, w0.capacities("src"))
    dc = kvt_amd.Cache(0, dst_layers, w0.capacities("dst"))
    slot = kvt_amd.PlanSlot(0, 1, w0.capacities("src"), w0.capacities("dst"), max_entries=16384,
                            chunk_bytes=chunk, max_layer_bytes=48 << 20)
    stride = 48 << 20
    packed = torch.zeros(w0.n_layers * stride, dtype=torch.uint8, device="cuda")
    stream = checkers.side_stream()
    kvt_amd.set_copy_cu_usage(0, usage)
    try:
        for w in ws:
            _check_eager(slot, w, sc, dc, src_layers, dst_layers, packed, stride, stream)
    finally:
        kvt_amd.set_copy_cu_usage(0, 1.0)
    # an empty batch moves nothing
    slot.fill(kvt_amd.BlockLists(), stream.cuda_stream)
    packed.fill_(7)
    torch.cuda.synchronize()
    slot.pack(sc, 0, w0.n_layers, packed, stride, stream.cuda_stream)
    stream.synchronize()
    assert bool((packed == 7).all())
    # an eager launch on another stream than the fill's orders itself behind the fill
    other = checkers.side_stream()
    lay = slot.fill(_lists(ws[1]), stream.cuda_stream)
    slot.pack(sc, 0, 1, packed, stride, other.cuda_stream)
    other.synchronize()
    blob = checkers.oracle_pack(_host(src_layers[0][0]), _oracle_lists(ws[1])[0])
    assert np.array_equal(_host(packed)[:len(blob)], blob) and lay.tensor_bytes[0] == len(blob)
    slot.close()


@pytest.mark.parametrize("chunk", [4096, 8192, 32768])
def test_two_tensors_per_layer(chunk):
    ws = [workloads.deepseek_mla(n_layers=2, pool=96, n_req=3, tokens=1000, seed=11),
          workloads.deepseek_mla(n_layers=2, pool=96, n_req=1, tokens=200, seed=12),
          workloads.deepseek_mla(n_layers=2, pool=96, n_req=5, tokens=640, seed=13)]
    w0 = ws[0]
    src_layers = _make_caches(w0, "src", 7)
    dst_layers = _make_caches(w0, "dst", 8, fill=False)
    sc = kvt_amd.Cache(0, src_layers, w0.capacities("src"))
    dc = kvt_amd.Cache(0, dst_layers, w0.capacities("dst"))
    slot = kvt_amd.PlanSlot(0, 2, w0.capacities("src"), w0.capacities("dst"), max_entries=4096,
                            chunk_bytes=chunk, max_layer_bytes=8 << 20)
    stride = 8 << 20
    packed = torch.zeros(w0.n_layers * stride, dtype=torch.uint8, device="cuda")
    stream = checkers.side_stream()
    offsets = set()
    for w in ws:
        offsets.add(_check_eager(slot, w, sc, dc, src_layers, dst_layers, packed, stride, stream).tensor_offset[1])
    assert len(offsets) == 3                           # the second blob moved with every batch
    slot.close()


@pytest.mark.parametrize("usage", [1.0, 0.25])
@pytest.mark.parametrize("heads,chunk", [(8, 0), (8, 16384), (2, 8192), (1, 4096)])
def test_transposing_slot(heads, chunk, usage):
    lib = checkers.oracle()
    ws = [workloads.llama70b_flashinfer(n_layers=2, pool=128, n_req=n, tokens=tok, seed=30 + n, heads=heads)
          for n, tok in ((3, 500), (1, 64), (4, 300))]
    w0 = ws[0]
    hd, ntpb, row = w0.xform
    B = 2 * hd * ntpb * row
    src_layers = _make_caches(w0, "src", 9)
    dst_layers = _make_caches(w0, "dst", 10, fill=False)
    sc = kvt_amd.Cache(0, src_layers, w0.capacities("src"))
    dc = kvt_amd.Cache(0, dst_layers, w0.capacities("dst"))
    slot = kvt_amd.PlanSlot(0, 1, w0.capacities("src"), w0.capacities("dst"), max_entries=16384,
                            xform=w0.xform, chunk_bytes=chunk, max_layer_bytes=16 << 20)
    stride = 16 << 20
    packed = torch.zeros(w0.n_layers * stride, dtype=torch.uint8, device="cuda")
    stream = checkers.side_stream()
    kvt_amd.set_copy_cu_usage(0, usage)
    try:
        for w in ws:
            lists = _lists(w)
            runs = lists.tensor(0)
            ids = np.concatenate([np.arange(r[0] // B, (r[0] + r[2]) // B) for r in runs]).astype(np.uint32)
            dst_ids = np.concatenate([np.arange(r[1] // B, (r[1] + r[2]) // B) for r in runs]).astype(np.uint32)
            lay = slot.fill(lists, stream.cuda_stream)
            for x in dst_layers:
                x[0].fill_(0xA5)
            torch.cuda.synchronize()
            slot.pack(sc, 0, w.n_layers, packed, stride, stream.cuda_stream)
            slot.unpack(dc, 0, w.n_layers, packed, stride, stream.cuda_stream)
            stream.synchronize()
            ph = _host(packed)
            for l in range(w.n_layers):
                hnd = _host(src_layers[l][0])
                blob = np.zeros(len(ids) * B, dtype=np.uint8)
                lib.kvto_pack_hnd_to_nhd(hnd.ctypes.data, ids.ctypes.data, len(ids), hd, ntpb, row,
                                         blob.ctypes.data)
                assert lay.tensor_bytes[0] == len(blob)
                assert np.array_equal(ph[l * stride:l * stride + len(blob)], blob), l
                exp = np.full(w.capacities("dst")[0], 0xA5, dtype=np.uint8)
                lib.kvto_unpack_nhd_to_hnd(exp.ctypes.data, dst_ids.ctypes.data, len(ids), hd, ntpb, row,
                                           blob.ctypes.data)
                assert np.array_equal(_host(dst_layers[l][0]), exp), l
    finally:
        kvt_amd.set_copy_cu_usage(0, 1.0)
    slot.close()


@pytest.mark.parametrize("usage", [1.0, 0.25])
@pytest.mark.parametrize("chunk", [0, 4096, 8192, 65536])
@pytest.mark.parametrize("layout,p_tp,d_tp,rank", [("flash", 2, 1, 1), ("ragged", 1, 2, 1), ("flash", 8, 1, 3)])
def test_run_slots_for_tp_split_batches(layout, p_tp, d_tp, rank, chunk, usage):
    def make(k, n_req, hi):
        return workloads.tp_split(layout, p_tp, d_tp, rank, n_layers=2, src_pool=96, dst_pool=144,
                                  n_req=n_req, min_tok=10, max_tok=hi, seed=50 + k)
    ws = [make(0, 4, 500), make(1, 1, 50), make(2, 7, 300)]
    w0 = ws[0]
    src_layers = _make_caches(w0, "src", 13)
    dst_layers = _make_caches(w0, "dst", 14, fill=False)
    sc = kvt_amd.Cache(0, src_layers, w0.capacities("src"))
    dc = kvt_amd.Cache(0, dst_layers, w0.capacities("dst"))
    slot = kvt_amd.PlanSlot(0, 1, w0.capacities("src"), w0.capacities("dst"), max_entries=16384,
                            chunk_bytes=chunk, max_layer_bytes=16 << 20, runs=True)
    stride = 16 << 20
    packed = torch.zeros(w0.n_layers * stride, dtype=torch.uint8, device="cuda")
    stream = checkers.side_stream()
    kvt_amd.set_copy_cu_usage(0, usage)
    try:
        for w in ws:
            src, dst = w.worker_infos()
            runs, _ = pipeline.parse_batch_runs(w.cache_shape, src, dst, w.task_bufs())
            _check_eager(slot, w, sc, dc, src_layers, dst_layers, packed, stride, stream, fill_with=runs)
            assert slot.num_strided_chunks > 0
    finally:
        kvt_amd.set_copy_cu_usage(0, 1.0)
    slot.close()


@pytest.mark.parametrize("chunk", [4096, 8192, 32768])
def test_converting_run_slot(chunk):
    from test_gpu_runs import _oracle_pack_fp8
    def make(k, n_req, hi):
        return workloads.tp_split("flash", 2, 1, 1, n_layers=2, src_pool=96, dst_pool=144, n_req=n_req,
                                  min_tok=10, max_tok=hi, seed=60 + k, fp8_dst=True)
    ws = [make(0, 4, 500), make(1, 1, 50), make(2, 6, 300)]
    w0 = ws[0]
    src_layers = _make_caches(w0, "src", 15)
    dst_layers = _make_caches(w0, "dst", 16, fill=False)
    sc = kvt_amd.Cache(0, src_layers, w0.capacities("src"))
    dc = kvt_amd.Cache(0, dst_layers, w0.capacities("dst"))
    slot = kvt_amd.PlanSlot(0, 1, w0.capacities("src"), w0.capacities("dst"), max_entries=16384,
                            chunk_bytes=chunk, max_layer_bytes=8 << 20, runs=True, bf16_to_fp8=True)
    stride = 8 << 20
    packed = torch.zeros(w0.n_layers * stride, dtype=torch.uint8, device="cuda")
    stream = checkers.side_stream()
    for w in ws:
        src, dst = w.worker_infos()
        runs, _ = pipeline.parse_batch_runs(w.cache_shape, src, dst, w.task_bufs(), fp8=True)
        rc, valid, tps, tpr, pid, kind = checkers.oracle_select(w.cache_shape, src, dst)
        rc, outs = checkers.oracle_parse(pid, src, dst, valid, tps, tpr, w.task_bufs(), fp8=True)
        assert rc == 0
        ranges = np.ascontiguousarray(outs[0], dtype=np.uint64)
        lay = slot.fill(runs, stream.cuda_stream)
        for x in dst_layers:
            x[0].fill_(0xA5)
        torch.cuda.synchronize()
        slot.pack(sc, 0, w.n_layers, packed, stride, stream.cuda_stream)
        slot.unpack(dc, 0, w.n_layers, packed, stride, stream.cuda_stream)
        stream.synchronize()
        for l in range(w.n_layers):
            blob = _oracle_pack_fp8(_host(src_layers[l][0]), ranges)
            assert lay.tensor_bytes[0] == len(blob)
            assert np.array_equal(_host(packed)[l * stride:l * stride + len(blob)], blob), l
            exp = np.full(w.capacities("dst")[0], 0xA5, dtype=np.uint8)
            checkers.oracle_unpack(exp, ranges, blob)
            assert np.array_equal(_host(dst_layers[l][0]), exp), l
    slot.close()


def test_launch_checks_of_a_slot():
    w = _batch(1, 2, 200, n_layers=2)
    src_layers = _make_caches(w, "src", 5)
    sc = kvt_amd.Cache(0, src_layers, w.capacities("src"))
    slot = kvt_amd.PlanSlot(0, 1, w.capacities("src"), w.capacities("dst"), max_entries=1024,
                            max_layer_bytes=64 << 20)
    slot.fill(_lists(w))
    torch.cuda.empty_cache()                            # a segment of exactly the buffer's size
    packed = torch.zeros(2 * (64 << 20), dtype=torch.uint8, device="cuda")
    with pytest.raises(kvt_amd.KvtError) as e:          # a stride below the room the slot was made for
        slot.pack(sc, 0, 2, packed, 32 << 20)
    assert "layer_stride" in str(e.value)
    with pytest.raises(kvt_amd.KvtError) as e:          # misaligned buffer
        slot.pack(sc, 0, 1, packed.data_ptr() + 4, 64 << 20)
    assert "16-byte" in str(e.value)
    with pytest.raises(kvt_amd.KvtError) as e:          # room for one layer only behind this address
        slot.pack(sc, 0, 2, packed.data_ptr() + (64 << 20), 64 << 20)
    assert "packed buffer" in str(e.value)
    with pytest.raises(kvt_amd.KvtError) as e:
        slot.pack_at(sc, 0, 1, packed, 64 << 20, [0] * 8)
    assert "kvt_pack_at" in str(e.value)
    small = kvt_amd.Cache(0, [[x[0][:1 << 20]] for x in src_layers], [1 << 20])
    with pytest.raises(kvt_amd.KvtError):
        slot.pack(small, 0, 1, packed, 64 << 20)
    torch.cuda.synchronize()
    slot.close()


class _Transport(threading.Thread):
    """The sender's thread: for every (step, layer) wait for the layer, then fetch its packed
    bytes on this thread's own stream, with no other synchronisation."""

    def __init__(self, sess, packed, stride, n_layers, lengths):
        super().__init__()
        self.sess, self.packed, self.stride, self.n_layers = sess, packed, stride, n_layers
        self.lengths = lengths                       # step -> bytes of a packed layer to fetch
        self.got, self.error = {}, None

    def run(self):
        try:
            stream = torch.cuda.Stream()
            for step in sorted(self.lengths):
                n = self.lengths[step]
                for l in range(self.n_layers):
                    self.sess.wait_layer(l, step)
                    host = torch.empty(max(n, 1), dtype=torch.uint8).pin_memory()
                    with torch.cuda.stream(stream):
                        host.copy_(self.packed[l * self.stride:l * self.stride + max(n, 1)], non_blocking=True)
                    stream.synchronize()
                    self.got[(step, l)] = host.numpy()[:n].copy()
                self.done_step = step
        except Exception as e:                       # noqa: BLE001 - handed to the main thread
            self.error = e


@pytest.mark.parametrize("usage", [1.0, 0.25], ids=["unlimited", "quarter"])
def test_one_captured_graph_packs_a_new_batch_on_every_replay(usage):
    """Capture the per-layer sequence of a session ONCE (forward pass stand-in, save_layer per
    layer) and a graph of per-layer unpack launches on the receiving side; then replay them for
    six batches with different block tables and request counts -- among them an empty batch and
    one that takes every table entry. A transport thread waits per layer and must find the
    blob of THAT replay's lists; the unpacked cache must equal the oracle's for that batch. A
    batch beyond the capacity is refused on the host and the slot keeps what it held."""
    n_layers = 4
    ws = [_batch(21, 5, 1200, n_layers), _batch(22, 1, 64, n_layers), None,
          _batch(23, 12, 600, n_layers), _batch(24, 2, 3000, n_layers), _batch(25, 8, 900, n_layers)]
    w0 = ws[0]
    s_cap, d_cap = w0.capacities("src"), w0.capacities("dst")
    all_lists = [(_lists(w) if w is not None else kvt_amd.BlockLists()) for w in ws]
    need = [kvt_amd.Plan(-1, l, s_cap, d_cap, chunk_bytes=32768).num_chunks if w is not None else 0
            for l, w in zip(all_lists, ws)]
    capacity = max(need)                              # the largest batch takes every entry
    room = max(kvt_amd.Plan(-1, l, s_cap, d_cap).layer_bytes for l, w in zip(all_lists, ws) if w is not None)
    src_layers = _make_caches(w0, "src", 31)
    staging = [[torch.zeros_like(x[0])] for x in src_layers]
    dst_layers = _make_caches(w0, "dst", 32, fill=False)
    sc = kvt_amd.Cache(0, src_layers, s_cap)
    dc = kvt_amd.Cache(0, dst_layers, d_cap)
    send = kvt_amd.PlanSlot(0, 1, s_cap, d_cap, max_entries=capacity, max_layer_bytes=room)
    recv = kvt_amd.PlanSlot(0, 1, s_cap, d_cap, max_entries=capacity, max_layer_bytes=room)
    stride = room
    packed = torch.zeros(n_layers * stride, dtype=torch.uint8, device="cuda")
    kvt_amd.set_copy_cu_usage(0, usage)
    try:
        sess = kvt_amd.Session(send, sc, packed, stride)
        s = checkers.side_stream()
        graph, ungraph = torch.cuda.CUDAGraph(), torch.cuda.CUDAGraph()
        blocks_before = kvt_amd.copy_ticket_stats(0)
        with torch.cuda.stream(s):
            with torch.cuda.graph(graph, stream=s):
                for l in range(n_layers):
                    src_layers[l][0].copy_(staging[l][0])       # the "forward pass" writes layer l
                    sess.save_layer(l, s.cuda_stream)
                    torch.cuda._sleep(2_000_000)
                sess.join(s.cuda_stream)
            with torch.cuda.graph(ungraph, stream=s):
                for l in range(n_layers):
                    recv.unpack(dc, l, 1, packed.data_ptr() + l * stride, stride, s.cuda_stream)
        # the per-layer launches of a capture are a chain of kernel nodes: they share ONE block of
        # work counters per plan, capture and stream instead of holding one each for good
        blocks_after = kvt_amd.copy_ticket_stats(0)
        assert blocks_after[2] - blocks_before[2] == 2 and blocks_after[3] == blocks_before[3]
    finally:
        kvt_amd.set_copy_cu_usage(0, 1.0)
    # once launches of the session have been captured, only its own slot may be named again
    sess.set_plan(send, packed, stride)
    other = kvt_amd.Plan(0, all_lists[0], s_cap, d_cap)
    with pytest.raises(kvt_amd.KvtError):
        sess.set_plan(other, packed, stride)
    lengths = {}
    o_lists = [(_oracle_lists(w)[0] if w is not None else np.zeros((0, 3), np.uint64)) for w in ws]
    for k in range(len(ws)):
        lengths[k + 1] = int(o_lists[k][:, 2].sum())
    transport = _Transport(sess, packed, stride, n_layers, lengths)
    transport.start()
    for k, w in enumerate(ws):
        contents = [_dev_bytes(s_cap[0], 700 + 10 * k + l, "u8") for l in range(n_layers)]
        with torch.cuda.stream(s):
            for l in range(n_layers):
                staging[l][0].copy_(contents[l])
                dst_layers[l][0].fill_(0xA5)
        lay = send.fill(all_lists[k], s.cuda_stream)
        assert lay.n_entries == need[k] and lay.tensor_bytes[0] == lengths[k + 1]
        if k == 3:                                    # a batch too large for the table: refused, nothing changes
            big = kvt_amd.BlockLists()
            big.append(0, np.concatenate([all_lists[k].tensor(0), [[0, 0, 4096]]]))
            with pytest.raises(kvt_amd.KvtError) as e:
                send.fill(big, s.cuda_stream)
            assert e.value.code == kvt_amd.ctypes_defs.ERR_OUT_OF_RANGE
            assert send.num_chunks == need[k]
        step = sess.begin_step()
        assert step == k + 1
        with torch.cuda.stream(s):
            graph.replay()
        # the receiving side: the same lists arrive, its slot is refilled, its graph replayed
        # once the transport has the whole step (the next replay overwrites the packed buffer)
        deadline = time.time() + 60
        while getattr(transport, "done_step", 0) < step and transport.error is None:
            assert time.time() < deadline
            time.sleep(0.0005)
        recv.fill(all_lists[k], s.cuda_stream)
        with torch.cuda.stream(s):
            ungraph.replay()
        s.synchronize()
        for l in range(n_layers):
            blob = checkers.oracle_pack(_host(contents[l]), o_lists[k])
            assert np.array_equal(transport.got[(step, l)], blob), (k, l)
            exp = np.full(d_cap[0], 0xA5, dtype=np.uint8)
            checkers.oracle_unpack(exp, o_lists[k], blob)
            assert np.array_equal(_host(dst_layers[l][0]), exp), (k, l)
    transport.join(60)
    assert not transport.is_alive()
    if transport.error is not None:
        raise transport.error
    sess.close()
    other.close()
    send.close()
    recv.close()


def test_the_host_may_run_one_fill_ahead_of_the_device():
    """Fills and replays queued back to back without waiting: fill k+1 is built while replay k
    runs (two staging copies in turn); every replay still packs its own batch."""
    n_layers = 2
    ws = [_batch(40 + k, 2 + 3 * (k % 3), 400 + 300 * (k % 4), n_layers) for k in range(8)]
    w0 = ws[0]
    s_cap, d_cap = w0.capacities("src"), w0.capacities("dst")
    src_layers = _make_caches(w0, "src", 33)
    sc = kvt_amd.Cache(0, src_layers, s_cap)
    slot = kvt_amd.PlanSlot(0, 1, s_cap, d_cap, max_entries=8192, max_layer_bytes=32 << 20)
    stride = 32 << 20
    outs = [torch.zeros(n_layers * stride, dtype=torch.uint8, device="cuda") for _ in ws]
    packed = torch.zeros(n_layers * stride, dtype=torch.uint8, device="cuda")
    s = checkers.side_stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(s):
        with torch.cuda.graph(graph, stream=s):
            slot.pack(sc, 0, n_layers, packed, stride, s.cuda_stream)
    lists = [_lists(w) for w in ws]
    with torch.cuda.stream(s):
        torch.cuda._sleep(50_000_000)                # the device falls behind the host
        for k in range(len(ws)):
            slot.fill(lists[k], s.cuda_stream)
            graph.replay()
            outs[k].copy_(packed, non_blocking=True)
    s.synchronize()
    for k, w in enumerate(ws):
        o = _oracle_lists(w)[0]
        for l in range(n_layers):
            blob = checkers.oracle_pack(_host(src_layers[l][0]), o)
            assert np.array_equal(_host(outs[k])[l * stride:l * stride + len(blob)], blob), (k, l)
    slot.close()
