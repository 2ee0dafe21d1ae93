"""The reference's end-to-end test of this path, replayed on the library:
KVTransferClientTest.TestKernelSyncAndDataTransfer
(kvtransfer/tests/client_step_test.cu:103-206). Two layers of 128 blocks x 16 KiB
are produced by kernels on a compute stream, each followed by an event; one
request (64 tokens, source blocks 0..3 -> destination blocks 4..7) is sent
layer by layer through a channel into *host* layers; every destination block of
layer 0 must sum to 10 x block_size and of layer 1 to 20 x block_size. The
reference plugs in a FakeChannel that copies range by range; here the channel is
kvt_amd.channel.LoopbackChannel (one pack + one unpack launch per layer, gated
on the layer's event on a side stream). Needs a real MI355X."""
import numpy as np
import pytest

import checkers
import kvt_amd
from kvt_amd import pipeline
from kvt_amd.channel import LoopbackChannel
from kvt_amd.ctypes_defs import SHAPE_RAGGED_FLASH, TaskBuf, make_worker_info

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

KB = 1024


def test_kernel_sync_and_data_transfer():
    num_layers, block_size, nblk = 2, 16 * KB, 128
    data_size = nblk * block_size
    stream = checkers.side_stream()
    layers = [torch.zeros(data_size, dtype=torch.uint8, device="cuda") for _ in range(num_layers)]
    host_layers = [torch.zeros(data_size, dtype=torch.uint8, pin_memory=True)
                   for _ in range(num_layers)]
    info = dict(block_sizes=[block_size], token_sizes=[KB], layer_num_blocks=nblk, tp=1, rank=0,
                num_layers=num_layers)
    src_info, dst_info = make_worker_info(**info), make_worker_info(**info)
    dst_blocks = [4, 5, 6, 7]
    # submit_req_send("0", 0, REQ, seen=0, new=16*4, last=true, {{0,1,2,3}}, dst_blocks)
    task = TaskBuf(0, 16 * 4, True, [[0, 1, 2, 3]], [dst_blocks])
    lists, tp_kind = pipeline.parse_batch(SHAPE_RAGGED_FLASH, src_info, dst_info, [task])

    src_cache = kvt_amd.Cache(0, [[l] for l in layers], [data_size])
    dst_cache = kvt_amd.Cache(0, [[h] for h in host_layers], [data_size])
    ch = LoopbackChannel(0, src_cache, dst_cache, [data_size], [data_size])
    ch.connect(dst_info)
    assert ch.is_active()
    ch.register_data(lists, tp_kind, num_layers,
                     lambda n: torch.zeros(n, dtype=torch.uint8, device="cuda"))
    torch.cuda.synchronize()          # what the default stream still holds comes first
    with torch.cuda.stream(stream):
        layers[0].fill_(10)                       # mock layer 0
        ch.send_data(0, stream.cuda_stream)       # event record + notify_event_record
        layers[1].fill_(20)                       # mock layer 1
        ch.send_data(1, stream.cuda_stream)
    stream.synchronize()
    metrics = ch.flush()
    assert "layers_sent=2," in metrics and "sb_size_total=%d," % (4 * block_size) in metrics

    for layer, val in ((0, 10), (1, 20)):
        host = host_layers[layer].numpy()
        for bid in dst_blocks:
            blk = host[bid * block_size:(bid + 1) * block_size]
            assert int(blk.astype(np.uint32).sum()) == val * block_size
        untouched = np.delete(host.reshape(nblk, block_size), dst_blocks, axis=0)
        assert not untouched.any()
    ch.close()
    assert not ch.is_active()


def test_channel_rejects_metadata_beyond_the_destination():
    block_size, nblk = 16 * KB, 8
    info = dict(block_sizes=[block_size], token_sizes=[KB], layer_num_blocks=nblk, tp=1, rank=0)
    src_info, dst_info = make_worker_info(**info), make_worker_info(**info)
    lists, tp_kind = pipeline.parse_batch(SHAPE_RAGGED_FLASH, src_info, dst_info,
                                          [TaskBuf(0, 32, True, [[0, 1]], [[6, 7]])])
    layer = torch.zeros(nblk * block_size, dtype=torch.uint8, device="cuda")
    small = torch.zeros(7 * block_size, dtype=torch.uint8, device="cuda")   # receiver has 7 blocks
    sc = kvt_amd.Cache(0, [[layer]], [nblk * block_size])
    dc = kvt_amd.Cache(0, [[small]], [7 * block_size])
    ch = LoopbackChannel(0, sc, dc, [nblk * block_size], [7 * block_size])
    ch.connect(dst_info)
    with pytest.raises(kvt_amd.KvtError):
        ch.register_data(lists, tp_kind, 1, lambda n: torch.zeros(n, dtype=torch.uint8, device="cuda"))
    ch.close()


def test_cuda_kernel_sync_over_four_steps():
    """StepTest.TestCudaKernelSync (kvtransfer/tests/step_sync_test.cu:18-104): four steps,
    each filling layer 0 with step+1 and layer 1 with step+2 on a non-blocking stream; a
    consumer thread waits for each layer and must see the step's value in every byte. The
    reference's consumer blocks in Step::wait_layer_ready and copies the layer; here it blocks
    in kvt_session_wait_layer and reads the layer's packed copy."""
    import threading

    num_layers, data_size = 2, 128 * (1 << 14)
    stream = checkers.side_stream()
    layers = [torch.zeros(data_size, dtype=torch.uint8, device="cuda") for _ in range(num_layers)]
    lists = kvt_amd.BlockLists()
    lists.append(0, [(0, 0, data_size)])
    plan = kvt_amd.Plan(0, lists, [data_size], [data_size])
    cache = kvt_amd.Cache(0, [[l] for l in layers], [data_size])
    packed = torch.zeros(num_layers * plan.layer_bytes, dtype=torch.uint8, device="cuda")
    for step in range(4):
        session = kvt_amd.Session(plan, cache, packed, plan.layer_bytes)
        seen, errors = {}, []

        def consumer():
            try:
                for layer in range(num_layers):
                    session.wait_layer(layer)
                    got = packed[layer * plan.layer_bytes:][:data_size].cpu().numpy()
                    seen[layer] = (int(got[:128].max()), int(got[:128].min()),
                                   int(got.astype(np.uint64).sum()))
            except Exception as e:
                errors.append(e)

        t = threading.Thread(target=consumer)     # waits before the layers are even launched
        t.start()
        torch.cuda.synchronize()          # what the default stream still holds comes first
        with torch.cuda.stream(stream):
            layers[0].fill_(step + 1)
            session.save_layer(0, stream.cuda_stream)
            layers[1].fill_(step + 2)
            session.save_layer(1, stream.cuda_stream)
        stream.synchronize()
        t.join()
        assert not errors, errors
        for layer in range(num_layers):
            val = step + 1 + layer
            assert seen[layer] == (val, val, val * data_size), (step, layer, seen[layer])
        session.close()


def test_channel_with_a_tp_remapping_destination():
    """Same flow with the sender on TP2 and the receiver on TP1: the channel folds the
    per-token ranges into strided runs before planning."""
    import checkers
    from kvt_amd import workloads
    from test_gpu_pack import _host, _make_caches
    w = workloads.tp_split("flash", 2, 1, 1, n_layers=2, src_pool=200, dst_pool=300, n_req=3,
                           min_tok=40, max_tok=600)
    src_info, dst_info = w.worker_infos()
    lists, tp_kind = pipeline.parse_batch(w.cache_shape, src_info, dst_info, w.task_bufs())
    assert tp_kind != 0
    expect = lists.tensor(0)
    src_layers = _make_caches(w, "src", 81)
    dst_layers = _make_caches(w, "dst", 82, fill=False)
    sc = kvt_amd.Cache(0, src_layers, w.capacities("src"))
    dc = kvt_amd.Cache(0, dst_layers, w.capacities("dst"))
    ch = LoopbackChannel(0, sc, dc, w.capacities("src"), w.capacities("dst"))
    ch.connect(dst_info)
    ch.register_data(lists, tp_kind, w.n_layers,
                     lambda n: torch.zeros(n, dtype=torch.uint8, device="cuda"))
    assert ch.plan.num_strided_chunks > 0
    for l in range(w.n_layers):
        ch.send_data(l, None)
    ch.flush()
    for l in range(w.n_layers):
        exp = np.full(w.capacities("dst")[0], 0xA5, dtype=np.uint8)
        blob = checkers.oracle_pack(_host(src_layers[l][0]), expect)
        checkers.oracle_unpack(exp, expect, blob)
        assert np.array_equal(_host(dst_layers[l][0]), exp), l
    ch.close()
