"""GPU end-to-end tests of the layer messages: a sender frames a layer around a
blob the GPU packs (directly into the pinned frame, or into HBM followed by a
DMA copy into the frame), a receiver parses the frame and unpacks out of it.
Frames are compared byte for byte with the format oracle filled with the CPU
oracle's blobs. Also the per-block store objects. Needs a real MI355X."""
import os
import sys

import numpy as np
import pytest

import checkers
import kvt_amd
from kvt_amd import binding, pipeline, workloads
from kvt_amd.binding import WIRE_RDMA_STAGED, WIRE_TCP
from test_gpu_pack import _host, _make_caches, _oracle_lists

sys.path.insert(0, os.path.join(checkers.ROOT, "oracle"))
import kvt_wire_oracle as wo  # noqa: E402

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _expected_frames(w, fmt, o_lists, src_layers, reqid):
    frames = []
    for l in range(w.n_layers):
        tensors = [([tuple(int(v) for v in r) for r in o_lists[t]],
                    checkers.oracle_pack(_host(src_layers[l][t]), o_lists[t]).tobytes())
                   for t in range(w.n_tensors)]
        if fmt == WIRE_TCP:
            frames.append(wo.tcp_write(reqid, l, tensors))
        else:
            frames.append(wo.staged_write(reqid, l, *tensors[0]))
    return frames


@pytest.mark.parametrize("fmt,direct", [(WIRE_TCP, True), (WIRE_TCP, False),
                                        (WIRE_RDMA_STAGED, True), (WIRE_RDMA_STAGED, False)])
def test_framed_layers_sender_to_receiver(fmt, direct):
    if fmt == WIRE_TCP:   # two tensors per layer
        w = workloads.deepseek_mla(n_layers=3, pool=256, n_req=3, tokens=1100)
    else:
        w = workloads.llama8b_batch(n_layers=3, src_pool=256, dst_pool=320, n_req=4,
                                    min_tok=100, max_tok=700)
    reqid = 0xABCDEF0123
    plan, lists = pipeline.build_plan(w, 0)
    o_lists = _oracle_lists(w)
    src_layers = _make_caches(w, "src", 31)
    dst_layers = _make_caches(w, "dst", 32, fill=False)
    sc = kvt_amd.Cache(0, src_layers, w.capacities("src"))
    dc = kvt_amd.Cache(0, dst_layers, w.capacities("dst"))
    lay = binding.wire_layout_of(fmt, lists)
    frame_bytes = lay.total_bytes
    offs = list(lay.blob_offset)
    stager = kvt_amd.Stager(0, frame_bytes + 64, 2)
    stream = checkers.side_stream()
    dev_buf = torch.zeros(plan.layer_bytes, dtype=torch.uint8, device="cuda")
    sent = []
    # ---- sender
    for l in range(w.n_layers):
        slot = l % 2
        binding.wire_write_frame(fmt, stager.slot_ptr(slot), stager.slot_bytes, reqid, l, lists)
        if direct:    # the kernel writes the blob areas of the pinned frame
            plan.pack_at(sc, l, 1, stager.slot_ptr(slot), 0, offs, stream.cuda_stream)
            stream.synchronize()
        else:         # pack into HBM, DMA each blob into its place
            plan.pack(sc, l, 1, dev_buf, plan.layer_bytes, stream.cuda_stream)
            for t in range(w.n_tensors):
                stager.save_at(slot, offs[t], dev_buf.data_ptr() + plan.tensor_offset(t),
                               plan.tensor_bytes(t), stream.cuda_stream)
            stager.wait(slot)
        sent.append(stager.slot_array(slot, frame_bytes).tobytes())
    for l, exp in enumerate(_expected_frames(w, fmt, o_lists, src_layers, reqid)):
        assert sent[l] == exp, l
    # ---- receiver: a fresh plan from what the frame says
    for l in range(w.n_layers):
        slot = l % 2
        stager.slot_array(slot, frame_bytes)[:] = np.frombuffer(sent[l], np.uint8)
        rc, r2, l2, rlists, rlay = binding.wire_parse_frame(
            fmt, stager.slot_ptr(slot), frame_bytes, w.n_tensors)
        assert rc == 0 and (r2, l2) == (reqid, l)
        for t in range(w.n_tensors):
            assert binding.validate_bounds(rlists.tensor(t), w.capacities("dst")[t], 1)[0] == 0
        # the receiver never gathers: an unbounded source side makes the plan unpack-only
        rplan = kvt_amd.Plan(0, rlists, [2**64 - 1] * w.n_tensors, w.capacities("dst"))
        if direct:
            rplan.unpack_at(dc, l, 1, stager.slot_ptr(slot), 0, list(rlay.blob_offset),
                            stream.cuda_stream)
        else:
            for t in range(w.n_tensors):
                stager.load_at(slot, rlay.blob_offset[t],
                               dev_buf.data_ptr() + rplan.tensor_offset(t), rlay.blob_bytes[t],
                               stream.cuda_stream)
            rplan.unpack(dc, l, 1, dev_buf, rplan.layer_bytes, stream.cuda_stream)
        stream.synchronize()
        rplan.close()
    for l in range(w.n_layers):
        for t in range(w.n_tensors):
            exp = np.full(w.capacities("dst")[t], 0xA5, dtype=np.uint8)
            blob = checkers.oracle_pack(_host(src_layers[l][t]), o_lists[t])
            checkers.oracle_unpack(exp, o_lists[t], blob)
            assert np.array_equal(_host(dst_layers[l][t]), exp), (l, t)
    stager.close()


def test_pack_at_several_layers_with_a_stride_and_odd_offsets():
    w = workloads.deepseek_mla(n_layers=4, pool=128, n_req=2, tokens=900)
    plan, lists = pipeline.build_plan(w, 0)
    o_lists = _oracle_lists(w)
    src_layers = _make_caches(w, "src", 41)
    sc = kvt_amd.Cache(0, src_layers, w.capacities("src"))
    offs = [48, 48 + plan.tensor_bytes(0) + 7] + [0] * 6     # second blob byte-misaligned
    stride = offs[1] + plan.tensor_bytes(1) + 5
    out = torch.full((w.n_layers * stride,), 0x11, dtype=torch.uint8, device="cuda")
    plan.pack_at(sc, 0, w.n_layers, out, stride, offs)
    torch.cuda.synchronize()
    out_h = _host(out)
    exp = np.full(w.n_layers * stride, 0x11, dtype=np.uint8)
    for l in range(w.n_layers):
        for t in range(2):
            blob = checkers.oracle_pack(_host(src_layers[l][t]), o_lists[t])
            exp[l * stride + offs[t]: l * stride + offs[t] + len(blob)] = blob
    assert np.array_equal(out_h, exp)
    dst_layers = _make_caches(w, "dst", 42, fill=False)
    dc = kvt_amd.Cache(0, dst_layers, w.capacities("dst"))
    plan.unpack_at(dc, 0, w.n_layers, out, stride, offs)
    torch.cuda.synchronize()
    for l in range(w.n_layers):
        for t in range(2):
            e = np.full(w.capacities("dst")[t], 0xA5, dtype=np.uint8)
            checkers.oracle_unpack(e, o_lists[t], checkers.oracle_pack(_host(src_layers[l][t]),
                                                                       o_lists[t]))
            assert np.array_equal(_host(dst_layers[l][t]), e), (l, t)


def test_pack_at_refuses_blob_offsets_and_strides_that_wrap():
    """A blob offset or layer stride near 2^64 must not wrap into an extent that fits the buffer."""
    w = workloads.deepseek_mla(n_layers=2, pool=64, n_req=1, tokens=300)
    plan, _ = pipeline.build_plan(w, 0)
    sc = kvt_amd.Cache(0, _make_caches(w, "src", 43), w.capacities("src"))
    out = torch.zeros(2 * plan.layer_bytes, dtype=torch.uint8, device="cuda")
    for offs, stride in (([2**64 - 16, 0] + [0] * 6, plan.layer_bytes),
                         ([0, plan.tensor_bytes(0)] + [0] * 6, 2**64 - 256)):
        with pytest.raises(kvt_amd.KvtError) as err:
            plan.pack_at(sc, 0, 2, out, stride, offs)
        assert err.value.code == 1, str(err.value)
    torch.cuda.synchronize()


def _info(block_sizes, nblk, n_layers):
    w = kvt_amd.ctypes_defs.WorkerInfo()
    w.engine_tp_size, w.worker_tp_rank = 1, 0
    w.n_tensors = len(block_sizes)
    for i, b in enumerate(block_sizes):
        w.block_sizes[i] = b
        w.token_sizes[i] = b // 16
    w.layer_num_blocks = nblk
    w.num_layers = n_layers
    return w


def test_block_objects_save_and_load_equal_kvcache_colon_blkid():
    """What FileBackend stores per (block, layer) is kvcache[:, blkid] (file_backend.py:279)
    and loading assigns it back (:232): objects packed by the GPU equal torch's own slices."""
    n_layers, nblk, bs, h, d = 3, 40, 16, 4, 64
    g = torch.Generator(device="cuda")
    g.manual_seed(77)
    kv = [torch.randn((2, nblk, bs, h, d), generator=g, device="cuda").to(torch.bfloat16)
          for _ in range(n_layers)]
    new = [torch.zeros_like(k) for k in kv]
    B = 2 * bs * h * d * 2
    rng = np.random.default_rng(3)
    src_ids = rng.permutation(nblk)[:17]
    dst_ids = rng.permutation(nblk)[:17]
    info = _info([B], nblk, n_layers)
    lists, ob = kvt_amd.block_object_lists(kvt_amd.ctypes_defs.SHAPE_FLASH, info, info, src_ids,
                                           dst_ids)
    plan = kvt_amd.Plan(0, lists, [B * nblk], [B * nblk])
    sc = kvt_amd.Cache(0, [[k.view(torch.uint8).reshape(-1)] for k in kv], [B * nblk])
    dc = kvt_amd.Cache(0, [[k.view(torch.uint8).reshape(-1)] for k in new], [B * nblk])
    assert plan.layer_bytes == len(src_ids) * ob
    objs = torch.zeros((n_layers, len(src_ids), ob), dtype=torch.uint8, device="cuda")
    plan.pack(sc, 0, n_layers, objs, plan.layer_bytes)
    torch.cuda.synchronize()
    for l in range(n_layers):
        for i, b in enumerate(src_ids):
            ref_obj = kv[l][:, int(b)].contiguous().view(torch.uint8).reshape(-1)
            assert torch.equal(objs[l, i], ref_obj), (l, i)
    plan.unpack(dc, 0, n_layers, objs, plan.layer_bytes)
    torch.cuda.synchronize()
    for l in range(n_layers):
        exp = torch.zeros_like(kv[l])
        exp[:, torch.as_tensor(dst_ids, device="cuda")] = kv[l][:, torch.as_tensor(src_ids, device="cuda")]
        assert torch.equal(new[l].view(torch.int16), exp.view(torch.int16)), l


def test_framed_layers_of_a_tp_remapping_batch_with_run_plans():
    """Sender: ParseBlock in run form, frame metadata = the expanded ranges, blob packed by the
    strided kernel straight into the pinned frame. Receiver: ranges off the frame folded back
    into runs, unpack straight out of the frame (blob at 4 or 12 modulo 16: word-wise path)."""
    w = workloads.tp_split("flash", 2, 1, 1, n_layers=2, src_pool=160, dst_pool=240, n_req=3,
                           min_tok=60, max_tok=500)
    src, dst = w.worker_infos()
    rc, valid, tps, tpr, pid, kind = checkers.oracle_select(w.cache_shape, src, dst)
    rc, outs = checkers.oracle_parse(pid, src, dst, valid, tps, tpr, w.task_bufs())
    assert rc == 0 and kind != 0
    o_runs = outs[0]
    plan, runs = pipeline.build_plan_runs(w, 0)
    lists = runs.expand()
    assert np.array_equal(lists.tensor(0), o_runs)
    src_layers = _make_caches(w, "src", 91)
    dst_layers = _make_caches(w, "dst", 92, fill=False)
    sc = kvt_amd.Cache(0, src_layers, w.capacities("src"))
    dc = kvt_amd.Cache(0, dst_layers, w.capacities("dst"))
    lay = binding.wire_layout_of(WIRE_RDMA_STAGED, lists)
    assert lay.blob_offset[0] % 16 in (4, 12)
    stager = kvt_amd.Stager(0, lay.total_bytes, 2)
    stream = checkers.side_stream()
    for l in range(w.n_layers):
        slot = l % 2
        binding.wire_write_frame(WIRE_RDMA_STAGED, stager.slot_ptr(slot), stager.slot_bytes, 7, l,
                                 lists)
        plan.pack_at(sc, l, 1, stager.slot_ptr(slot), 0, list(lay.blob_offset), stream.cuda_stream)
        stream.synchronize()
        frame = stager.slot_array(slot, lay.total_bytes).tobytes()
        blob = checkers.oracle_pack(_host(src_layers[l][0]), o_runs)
        assert frame == wo.staged_write(7, l, [tuple(int(v) for v in r) for r in o_runs],
                                        blob.tobytes())
        # receiver
        rc, reqid, layer, rlists, rlay = binding.wire_parse_frame(
            WIRE_RDMA_STAGED, stager.slot_ptr(slot), lay.total_bytes, 1)
        assert rc == 0 and (reqid, layer) == (7, l)
        rplan = kvt_amd.Plan(0, kvt_amd.RunLists.compress(rlists), [2**64 - 1],
                             w.capacities("dst"))
        assert rplan.num_strided_chunks > 0
        rplan.unpack_at(dc, l, 1, stager.slot_ptr(slot), 0, list(rlay.blob_offset),
                        stream.cuda_stream)
        stream.synchronize()
        exp = np.full(w.capacities("dst")[0], 0xA5, dtype=np.uint8)
        checkers.oracle_unpack(exp, o_runs, blob)
        assert np.array_equal(_host(dst_layers[l][0]), exp), l
        rplan.close()
    stager.close()


def test_per_block_objects_spanning_all_layers():
    """One pack launch builds, for every block, one object holding that block of all layers
    ([layer][K block][V block]); checked against torch.stack of kvcache[:, b] per layer, and
    loaded back into other blocks of a second cache."""
    n_layers, nblk, bs, h, d = 4, 24, 16, 2, 64
    g = torch.Generator(device="cuda")
    g.manual_seed(123)
    kv = [torch.randn((2, nblk, bs, h, d), generator=g, device="cuda").to(torch.bfloat16)
          for _ in range(n_layers)]
    new = [torch.zeros_like(k) for k in kv]
    B = 2 * bs * h * d * 2
    rng = np.random.default_rng(9)
    src_ids, dst_ids = rng.permutation(nblk)[:7], rng.permutation(nblk)[:7]
    info = kvt_amd.ctypes_defs.make_worker_info(block_sizes=[B], token_sizes=[B // bs],
                                                layer_num_blocks=nblk, num_layers=n_layers)
    lists, ob = kvt_amd.block_object_lists(kvt_amd.ctypes_defs.SHAPE_FLASH, info, info, src_ids,
                                           dst_ids)
    assert ob == B
    stride = n_layers * ob
    plan = kvt_amd.Plan(0, lists, [B * nblk], [B * nblk], objects=(ob, stride))
    sc = kvt_amd.Cache(0, [[k.view(torch.uint8).reshape(-1)] for k in kv], [B * nblk])
    dc = kvt_amd.Cache(0, [[k.view(torch.uint8).reshape(-1)] for k in new], [B * nblk])
    objs = torch.zeros((len(src_ids), stride), dtype=torch.uint8, device="cuda")
    plan.pack(sc, 0, n_layers, objs, ob)             # layer_stride = one layer's part
    torch.cuda.synchronize()
    for i, b in enumerate(src_ids):
        want = torch.stack([kv[l][:, int(b)] for l in range(n_layers)]).contiguous()
        assert torch.equal(objs[i], want.view(torch.uint8).reshape(-1)), i
    plan.unpack(dc, 0, n_layers, objs, ob)
    torch.cuda.synchronize()
    s_idx = torch.as_tensor(src_ids, device="cuda")
    d_idx = torch.as_tensor(dst_ids, device="cuda")
    for l in range(n_layers):
        exp = torch.zeros_like(kv[l])
        exp[:, d_idx] = kv[l][:, s_idx]
        assert torch.equal(new[l].view(torch.int16), exp.view(torch.int16)), l
