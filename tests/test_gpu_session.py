"""The per-layer completion signal of a session (kvt_session_*; the reference's Step /
StepGuard / CudaEventBarrier, kvtransfer/src/step.cpp:49-69, kvtransfer/src/context.cpp:18-20,
consumed by do_send, kvtransfer/src/tx_stub.cpp:395-415): "wait(L) returns once layer L of
this step is ready", for a transport thread beside the forward pass -- also when the forward
pass, the packs and their signals are ONE captured hipGraph that is only ever replayed.
No test here synchronises the device: the waiting thread learns about a layer from the
session alone and fetches that layer's bytes on a stream of its own. Needs a real MI355X."""
import threading
import time

import numpy as np
import pytest

import checkers
import kvt_amd
from kvt_amd import ctypes_defs, pipeline, workloads

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _contents(cap, seed):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    return torch.randint(0, 256, (cap,), generator=g, device="cuda", dtype=torch.uint8)


class _Transport(threading.Thread):
    """Stands where the reference's per-destination send thread stands: for every step and
    every layer, wait for the layer, then take its packed bytes (here: into pinned memory, on
    this thread's own stream)."""

    def __init__(self, sess, packed, stride, blob_len, n_layers, steps):
        super().__init__()
        self.sess, self.packed, self.stride, self.blob_len = sess, packed, stride, blob_len
        self.n_layers, self.steps = n_layers, steps
        self.got, self.returned_at, self.error = {}, {}, None

    def run(self):
        try:
            stream = checkers.side_stream()
            for step in self.steps:
                for l in range(self.n_layers):
                    self.sess.wait_layer(l, step)
                    self.returned_at[(step, l)] = time.perf_counter()
                    host = torch.empty(self.blob_len, dtype=torch.uint8).pin_memory()
                    # straight after the wait, on this thread's stream alone: the rest of the
                    # step or replay is still running, so equal bytes mean the layer was
                    # complete when the wait returned
                    with torch.cuda.stream(stream):
                        host.copy_(self.packed[l * self.stride:l * self.stride + self.blob_len],
                                   non_blocking=True)
                    stream.synchronize()           # this thread's stream only
                    self.got[(step, l)] = host.numpy().copy()
        except Exception as e:                     # noqa: BLE001 - handed to the main thread
            self.error = e


def test_graph_replays_signal_every_layer_to_a_waiting_thread():
    """Capture once, replay four times with different cache contents. The transport thread is
    started before the first replay, waits for (step, layer) pairs it knows in advance, and
    must find, each time, the bytes of THAT replay (an early return on stale state would show
    the previous replay's). A sleep kernel between the layers keeps them milliseconds apart,
    so layer 0's wait is seen to return while the graph is still running."""
    w = workloads.llama8b_single(n_layers=4, pool=64, tokens=200)
    plan, lists = pipeline.build_plan(w, 0)
    cap = w.capacities("src")[0]
    layers = [[torch.zeros(cap, dtype=torch.uint8, device="cuda")] for _ in range(w.n_layers)]
    staging = [torch.zeros(cap, dtype=torch.uint8, device="cuda") for _ in range(w.n_layers)]
    cache = kvt_amd.Cache(0, layers, [cap])
    stride = plan.layer_bytes
    blob_len = plan.tensor_bytes(0)
    packed = torch.zeros(w.n_layers * stride, dtype=torch.uint8, device="cuda")
    sess = kvt_amd.Session(plan, cache, packed, stride)
    graph = torch.cuda.CUDAGraph()
    s = checkers.side_stream()
    torch.cuda.synchronize()          # what the default stream still holds comes first
    with torch.cuda.stream(s):
        with torch.cuda.graph(graph, stream=s):
            for l in range(w.n_layers):
                layers[l][0].copy_(staging[l])          # the "forward pass" writes layer l
                sess.save_layer(l, s.cuda_stream)
                torch.cuda._sleep(10_000_000)           # some milliseconds of other work
            sess.join(s.cuda_stream)
    n_replays = 4
    transport = _Transport(sess, packed, stride, blob_len, w.n_layers, range(1, n_replays + 1))
    transport.start()
    expected, still_running = {}, []
    for rep in range(n_replays):
        contents = [_contents(cap, 900 + 10 * rep + l) for l in range(w.n_layers)]
        torch.cuda.synchronize()          # what the default stream still holds comes first
        with torch.cuda.stream(s):                      # eager work between the replays
            for l in range(w.n_layers):
                staging[l].copy_(contents[l])
        step = sess.begin_step()
        assert step == rep + 1
        finished = torch.cuda.Event()
        torch.cuda.synchronize()          # what the default stream still holds comes first
        with torch.cuda.stream(s):
            graph.replay()
            finished.record(s)
        deadline = time.time() + 60
        while (step, 0) not in transport.returned_at and transport.error is None:
            assert time.time() < deadline
            time.sleep(0.0001)
        still_running.append(not finished.query())
        for l in range(w.n_layers):
            expected[(step, l)] = checkers.oracle_pack(contents[l].cpu().numpy(), lists.tensor(0))
        # the next replay overwrites the packed buffer: let the transport take this step first
        # (what a real sender does by owning one buffer per step in flight)
        while (step, w.n_layers - 1) not in transport.got and transport.error is None:
            assert time.time() < deadline
            time.sleep(0.001)
    transport.join(60)
    assert not transport.is_alive()
    if transport.error is not None:
        raise transport.error
    for key, blob in expected.items():
        assert np.array_equal(transport.got[key], blob), key
    # layer 0 was reported while the rest of the graph was still on the GPU
    assert any(still_running), still_running
    for step in range(1, n_replays + 1):
        t = [transport.returned_at[(step, l)] for l in range(w.n_layers)]
        assert t == sorted(t)
        assert t[-1] - t[0] > 0.002, "the layers of a replay were reported together"
    s.synchronize()
    sess.close()


def test_eager_steps_share_one_session_and_waits_may_come_first():
    w = workloads.llama8b_batch(n_layers=5, src_pool=256, dst_pool=256, n_req=3, min_tok=200,
                                max_tok=900)
    plan, lists = pipeline.build_plan(w, 0)
    cap = w.capacities("src")[0]
    layers = [[torch.zeros(cap, dtype=torch.uint8, device="cuda")] for _ in range(w.n_layers)]
    cache = kvt_amd.Cache(0, layers, w.capacities("src"))
    stride = plan.layer_bytes
    blob_len = plan.tensor_bytes(0)
    packed = torch.zeros(w.n_layers * stride, dtype=torch.uint8, device="cuda")
    sess = kvt_amd.Session(plan, cache, packed, stride)
    compute = checkers.side_stream()
    transport = _Transport(sess, packed, stride, blob_len, w.n_layers, (1, 2, 3))
    transport.start()                                   # parks in wait_layer(0, step 1)
    time.sleep(0.05)
    for step in (1, 2, 3):
        fresh = [_contents(cap, 70 + 10 * step + l) for l in range(w.n_layers)]
        assert sess.begin_step() == step
        torch.cuda.synchronize()          # what the default stream still holds comes first
        with torch.cuda.stream(compute):
            for l in range(w.n_layers):
                layers[l][0].copy_(fresh[l])
                sess.save_layer(l, compute.cuda_stream)
        deadline = time.time() + 60
        while (step, w.n_layers - 1) not in transport.got and transport.error is None:
            assert time.time() < deadline
            time.sleep(0.001)
        if transport.error is not None:
            raise transport.error
        for l in range(w.n_layers):
            blob = checkers.oracle_pack(fresh[l].cpu().numpy(), lists.tensor(0))
            assert np.array_equal(transport.got[(step, l)], blob), (step, l)
    transport.join(60)
    assert not transport.is_alive() and transport.error is None
    # a step that has fallen out of the tracked window is refused, not waited for
    for _ in range(8):
        sess.begin_step()
    with pytest.raises(kvt_amd.KvtError) as e:
        sess.wait_layer(0, 3)
    assert "no longer tracked" in str(e.value)
    compute.synchronize()
    sess.close()


def test_a_failed_layer_wakes_the_waiting_thread_with_the_error():
    """The packed buffer is too short for the last layers: their launch is refused on the host
    (no kernel runs), the failure is latched in the step, and the thread that waits for such a
    layer returns that error instead of waiting for ever."""
    w = workloads.llama8b_single(n_layers=4, pool=64, tokens=200)
    plan, lists = pipeline.build_plan(w, 0)
    cap = w.capacities("src")[0]
    layers = [[_contents(cap, 5 + l)] for l in range(w.n_layers)]
    cache = kvt_amd.Cache(0, layers, [cap])
    stride = 64 << 20                                   # layers 64 MiB apart ...
    torch.cuda.empty_cache()                            # a segment of exactly that size
    packed = torch.zeros(2 * stride, dtype=torch.uint8, device="cuda")   # ... room for two
    sess = kvt_amd.Session(plan, cache, packed, stride)
    result = {}

    def waiter():
        try:
            sess.wait_layer(1, 1)
            result["layer1"] = "ok"
            sess.wait_layer(3, 1)
            result["layer3"] = "ok"
        except kvt_amd.KvtError as e:
            result["error"] = e

    t = threading.Thread(target=waiter)
    t.start()
    compute = checkers.side_stream()
    sess.begin_step()
    sess.save_layer(0, compute.cuda_stream)
    sess.save_layer(1, compute.cuda_stream)
    with pytest.raises(kvt_amd.KvtError) as refused:
        sess.save_layer(2, compute.cuda_stream)
    # beyond the allocation: "out of range", or "not device memory" where nothing is mapped there
    assert refused.value.code in (1, 3) and "packed buffer" in str(refused.value)
    t.join(30)
    assert not t.is_alive()
    assert "layer3" not in result
    assert result["error"].code == refused.value.code and "the step failed" in str(result["error"])
    # the next step starts clean
    sess.begin_step()
    sess.save_layer(0, compute.cuda_stream)
    sess.wait_layer(0)
    blob = checkers.oracle_pack(layers[0][0].cpu().numpy(), lists.tensor(0))
    assert np.array_equal(packed[:len(blob)].cpu().numpy(), blob)
    compute.synchronize()
    sess.close()


def test_destroying_a_session_releases_a_parked_waiter():
    w = workloads.llama8b_single(n_layers=2, pool=64, tokens=100)
    plan, _ = pipeline.build_plan(w, 0)
    cap = w.capacities("src")[0]
    layers = [[torch.zeros(cap, dtype=torch.uint8, device="cuda")] for _ in range(w.n_layers)]
    cache = kvt_amd.Cache(0, layers, [cap])
    packed = torch.zeros(w.n_layers * plan.layer_bytes, dtype=torch.uint8, device="cuda")
    sess = kvt_amd.Session(plan, cache, packed, plan.layer_bytes)
    result = {}

    def waiter():
        try:
            sess.wait_layer(1, 1)                       # never submitted
            result["returned"] = True
        except kvt_amd.KvtError as e:
            result["error"] = e

    t = threading.Thread(target=waiter)
    t.start()
    time.sleep(0.05)
    sess.close()
    t.join(30)
    assert not t.is_alive() and "returned" not in result
    assert "being destroyed" in str(result["error"])


def test_a_bounded_wait_runs_out_and_can_be_repeated():
    """kvt_session_wait_layer_for: a layer that is not there yet -- step not begun, layer not
    submitted -- gives KVT_ERR_TIMEOUT after the time given instead of parking the thread, and
    the same wait succeeds once the layer has been packed."""
    w = workloads.llama8b_single(n_layers=2, pool=64, tokens=100)
    plan, lists = pipeline.build_plan(w, 0)
    cap = w.capacities("src")[0]
    layers = [[_contents(cap, 70 + l)] for l in range(w.n_layers)]
    cache = kvt_amd.Cache(0, layers, [cap])
    packed = torch.zeros(w.n_layers * plan.layer_bytes, dtype=torch.uint8, device="cuda")
    sess = kvt_amd.Session(plan, cache, packed, plan.layer_bytes)
    compute = checkers.side_stream()
    for step, layer in ((1, 0), (3, 1)):             # step 1 has not begun; step 3 is far off
        t0 = time.perf_counter()
        with pytest.raises(kvt_amd.KvtError) as err:
            sess.wait_layer(layer, step, timeout_us=20_000)
        waited = time.perf_counter() - t0
        assert err.value.code == ctypes_defs.ERR_TIMEOUT, str(err.value)
        assert 0.015 < waited < 5.0, waited
    assert sess.begin_step() == 1
    sess.save_layer(0, compute.cuda_stream)
    with pytest.raises(kvt_amd.KvtError) as err:       # begun, but layer 1 not submitted
        sess.wait_layer(1, 1, timeout_us=5_000)
    assert err.value.code == ctypes_defs.ERR_TIMEOUT
    sess.wait_layer(0, 1, timeout_us=30_000_000)
    sess.save_layer(1, compute.cuda_stream)
    sess.wait_layer(1, 1, timeout_us=30_000_000)
    for l in range(w.n_layers):
        blob = checkers.oracle_pack(layers[l][0].cpu().numpy(), lists.tensor(0))
        got = packed[l * plan.layer_bytes:l * plan.layer_bytes + len(blob)].cpu().numpy()
        assert np.array_equal(got, blob), l
    compute.synchronize()
    sess.close()


def test_groups_of_layers_behind_one_event_eager_and_in_a_graph():
    """kvt_session_save_layers: several layers behind one event, packed by one launch; the
    transport still waits layer by layer. Eagerly with uneven groups, then the same groups
    captured once and replayed with other cache contents."""
    w = workloads.llama8b_single(n_layers=7, pool=96, tokens=700)
    plan, lists = pipeline.build_plan(w, 0)
    cap = w.capacities("src")[0]
    layers = [[_contents(cap, 200 + l)] for l in range(w.n_layers)]
    cache = kvt_amd.Cache(0, layers, [cap])
    stride = plan.layer_bytes
    packed = torch.zeros(w.n_layers * stride, dtype=torch.uint8, device="cuda")
    sess = kvt_amd.Session(plan, cache, packed, stride)
    ranges = lists.tensor(0)
    groups = [(0, 3), (3, 1), (4, 3)]
    with pytest.raises(kvt_amd.KvtError):
        sess.save_layers(5, 3)                                   # beyond the last layer
    with pytest.raises(kvt_amd.KvtError):
        sess.save_layers(2, 0)
    compute = checkers.side_stream()

    def check(step):
        t = _Transport(sess, packed, stride, plan.tensor_bytes(0), w.n_layers, [step])
        t.start()
        return t

    step = sess.begin_step()
    t = check(step)
    for first, n in groups:
        sess.save_layers(first, n, compute.cuda_stream)
    t.join(60)
    assert not t.is_alive() and t.error is None, t.error
    for l in range(w.n_layers):
        assert np.array_equal(t.got[(step, l)], checkers.oracle_pack(layers[l][0].cpu().numpy(), ranges)), l
    compute.synchronize()
    sess.close()

    sess = kvt_amd.Session(plan, cache, packed, stride)
    graph = torch.cuda.CUDAGraph()
    cap_stream = checkers.side_stream()
    with torch.cuda.graph(graph, stream=cap_stream):
        for first, n in groups:
            sess.save_layers(first, n, cap_stream.cuda_stream)
        sess.join(cap_stream.cuda_stream)
    for rep in range(3):
        for l in range(w.n_layers):
            layers[l][0].copy_(_contents(cap, 300 + 10 * rep + l))
        torch.cuda.synchronize()
        expect = [checkers.oracle_pack(layers[l][0].cpu().numpy(), ranges) for l in range(w.n_layers)]
        step = sess.begin_step()
        t = check(step)
        graph.replay()
        t.join(60)
        assert not t.is_alive() and t.error is None, t.error
        for l in range(w.n_layers):
            assert np.array_equal(t.got[(step, l)], expect[l]), (rep, l)
    torch.cuda.synchronize()
    sess.close()


def test_last_layers_packed_on_the_compute_stream_itself():
    """kvt_session_save_layers_inline: no hop to the side stream; same signal, same bytes, and
    the session may be destroyed while such a pack is still queued."""
    w = workloads.llama8b_single(n_layers=5, pool=96, tokens=600)
    plan, lists = pipeline.build_plan(w, 0)
    cap = w.capacities("src")[0]
    layers = [[_contents(cap, 400 + l)] for l in range(w.n_layers)]
    cache = kvt_amd.Cache(0, layers, [cap])
    stride = plan.layer_bytes
    packed = torch.zeros(w.n_layers * stride, dtype=torch.uint8, device="cuda")
    sess = kvt_amd.Session(plan, cache, packed, stride)
    compute = checkers.side_stream()
    for rep in range(2):
        step = sess.begin_step()
        t = _Transport(sess, packed, stride, plan.tensor_bytes(0), w.n_layers, [step])
        t.start()
        for l in range(3):
            sess.save_layer(l, compute.cuda_stream)
        sess.save_layers_inline(3, 2, compute.cuda_stream)
        t.join(60)
        assert not t.is_alive() and t.error is None, t.error
        for l in range(w.n_layers):
            blob = checkers.oracle_pack(layers[l][0].cpu().numpy(), lists.tensor(0))
            assert np.array_equal(t.got[(step, l)], blob), (rep, l)
    sess.begin_step()
    sess.save_layers_inline(0, w.n_layers, compute.cuda_stream)
    sess.close()                       # waits for the pack queued on the compute stream
    compute.synchronize()
