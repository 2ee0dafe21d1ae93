#!/usr/bin/env python3
"""Benchmark of the KV-cache pack/unpack hot path on one MI355X.

One *step* = one pass of the hot path over one batch: ParseBlock for every
request of the batch, merge, plan upload, then ONE pack launch (all layers) and
ONE unpack launch (all layers). Inputs (caches, block tables) are resident
before the timed region. Steps are issued the way a serving loop issues them:
the host prepares step k+1 while the GPU still runs step k.

Prints one JSON line: the whole-job rate plus `roofline` (dominant kernel against the HBM
peak) and `cpu_baseline` (the CPU oracle on a bounded sample of the same batch).
"""
import argparse
import ctypes as C
import json
import os
import statistics
import sys
import time
import types

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path[:0] = [os.path.join(ROOT, "llumnix-kv_amd"), os.path.join(ROOT, "tests")]

HBM_PEAK = 8.0e12  # bytes/s, MI355X HBM3E

def log(*a):
    print(*a, file=sys.stderr, flush=True)


def build_workload(cfg, scale, variant=0):
    """variant (config 2 only): another batch on the same pools (other lengths, other block
    tables), for the legs that give a captured graph a new batch per replay."""
    from kvt_amd import workloads as W
    if cfg == 1:
        return [W.llama8b_single()]
    if cfg == 2:
        seed = 20252 + 1000 * variant
        if scale < 1.0:
            return [W.llama8b_batch(n_layers=max(2, int(32 * scale)),
                                    src_pool=max(1024, int(16384 * scale)),
                                    dst_pool=max(1536, int(24576 * scale)),
                                    n_req=max(2, int(64 * scale)),
                                    min_tok=max(64, int(1024 * scale)),
                                    max_tok=max(128, int(8192 * scale)), seed=seed)]
        return [W.llama8b_batch(seed=seed)]
    if cfg == 3:
        return [W.llama70b_flashinfer(n_layers=max(2, int(80 * scale)),
                                      pool=max(512, int(8192 * scale)),
                                      n_req=max(2, int(32 * scale)))]
    if cfg == 4:
        return [W.deepseek_mla(n_layers=max(2, int(61 * scale)), pool=max(512, int(4608 * scale)),
                               n_req=max(2, int(16 * scale)))]
    if cfg == 5:
        return [W.qwen3next_attn(n_layers=max(2, int(12 * scale)),
                                 pool=max(512, int(36864 * scale)), n_req=max(2, int(128 * scale))),
                W.qwen3next_gdn(n_layers=max(2, int(36 * scale)), slots=max(4, int(256 * scale)),
                                n_req=max(2, int(128 * scale)))]
    if cfg == 9:
        # config 5 in the reference's own arrangement: one tensor per full-attention layer with
        # uniform 2 MiB pages shared by attention and the GDN states in front of it
        return [W.qwen3next_uniform_pages(n_layers=max(2, int(12 * scale)),
                                          pool=max(16, int(1024 * scale)),
                                          n_req=max(2, int(128 * scale)))]
    if cfg == 10:
        # config 9's model between a TP2 prefill and a TP1 decode instance: attention rows
        # split per token, GDN conv rows per channel group, SSM states, tail fill
        return [W.qwen3next_tp_split(2, 1, 0, n_layers=max(2, int(12 * scale)),
                                     pool=max(16, int(1024 * scale)),
                                     n_req=max(2, int(128 * scale)))]
    if cfg in (6, 7, 8, 11):
        # TP-remapping batches (not among the baseline configurations): config 2's batch with
        # the sender on TP2 and the receiver on TP1 (6), TP1 -> TP2 on the ragged layout (7),
        # TP2 -> TP1 on FlashInfer HND pages (8: per-head rows, whole segments of 4 KiB),
        # TP8 -> TP1 (11: one KV head per sender, table entries of 4 KiB)
        layout, p_tp, d_tp = {6: ("flash", 2, 1), 7: ("ragged", 1, 2), 8: ("hnd", 2, 1),
                              11: ("flash", 8, 1)}[cfg]
        return [W.tp_split(layout, p_tp, d_tp, 0, n_layers=max(2, int(32 * scale)),
                           src_pool=max(1024, int(16384 * scale)),
                           dst_pool=max(1536, int(24576 * scale)), n_req=max(2, int(64 * scale)),
                           min_tok=max(64, int(1024 * scale)), max_tok=max(128, int(8192 * scale)))]
    raise SystemExit("unknown --config %r" % cfg)


class DeviceSide:
    """Caches and packed buffer of one workload, resident in HBM."""

    def __init__(self, torch, kvt, w, seed):
        self.w = w
        g = torch.Generator(device="cuda")
        self.src, self.dst = [], []
        for l in range(w.n_layers):
            row_s, row_d = [], []
            for t, (cs, cd) in enumerate(zip(w.capacities("src"), w.capacities("dst"))):
                g.manual_seed(seed * 100003 + l * 16 + t)
                if w.elem_dtype == "bf16":
                    x = torch.empty(cs // 2, dtype=torch.bfloat16, device="cuda")
                    step = 1 << 28
                    for o in range(0, x.numel(), step):  # bounded fp32 temporaries
                        n = min(step, x.numel() - o)
                        x[o:o + n] = torch.rand(n, generator=g, device="cuda") * 2 - 1
                    row_s.append(x.view(torch.uint8))
                elif w.elem_dtype == "fp8":
                    x = torch.randn(cs, generator=g, device="cuda").clamp_(-448, 448)
                    row_s.append(x.to(torch.float8_e4m3fn).view(torch.uint8))
                else:
                    row_s.append(torch.randn(cs // 4, generator=g, device="cuda").view(torch.uint8))
                row_d.append(torch.zeros(cd, dtype=torch.uint8, device="cuda"))
            self.src.append(row_s)
            self.dst.append(row_d)
        self.src_cache = kvt.Cache(0, self.src, w.capacities("src"))
        self.dst_cache = kvt.Cache(0, self.dst, w.capacities("dst"))


class stdout_to_stderr:
    """The compiled reference announces every environment variable it reads on stdout
    (kvtransfer/src/envcfg.cpp:15); this file's stdout carries exactly one JSON line."""

    def __enter__(self):
        sys.stdout.flush()
        self.saved = os.dup(1)
        os.dup2(2, 1)

    def __exit__(self, *exc):
        os.dup2(self.saved, 1)
        os.close(self.saved)


def ev_ms(lib, a, b):
    ms = C.c_float()
    rc = lib.kvt_event_elapsed_ms(a, b, C.byref(ms))
    assert rc == 0, lib.kvt_last_error()
    return ms.value

def leg_cpu(c, out):
    """Parity spot check of the GPU results and the CPU baseline (oracle) on a bounded sample."""
    torch, np, kvt, lib, args, pipeline = c.torch, c.np, c.kvt, c.lib, c.args, c.pipeline
    wls, sides, infos, tasks, first = c.wls, c.sides, c.infos, c.tasks, c.first
    strides, packed, stream, sh, new_event = c.strides, c.packed, c.stream, c.sh, c.new_event
    full_wls, full_sides, mixed = c.full_wls, c.full_sides, c.mixed
    import checkers
    w, side = full_wls[0], full_sides[0]      # (mixed mode: both halves of the requests)
    L = max(1, min(args.cpu_layers, w.n_layers))
    if w.xform is not None:
        L = min(L, 4)      # the row-by-row permutation is several times slower than a memcpy
    s_info, d_info = w.worker_infos()
    cpu_tasks = w.task_bufs()
    rc, valid, tps, tpr, pid, kind = checkers.oracle_select(w.cache_shape, s_info, d_info)
    assert rc == 0
    olib = checkers.oracle()
    host_src = [[t.cpu().numpy() for t in side.src[l]] for l in range(L)]
    host_dst = [[np.zeros(c, dtype=np.uint8) for c in w.capacities("dst")] for _ in range(L)]
    stride = strides[0]
    gpu_packed = packed[0][:L * stride].cpu().numpy()
    plan0 = first[0][0]

    def cpu_pass():
        t_a = time.perf_counter()
        rc, outs = checkers.oracle_parse(pid, s_info, d_info, valid, tps, tpr, cpu_tasks)
        assert rc == 0
        if kind == 0:
            outs = [checkers.oracle_merge(o)[0] for o in outs]
        t_b = time.perf_counter()
        blobs = []
        if w.xform is None:
            for l in range(L):
                blobs.append([checkers.oracle_pack(host_src[l][t], outs[t])
                              for t in range(w.n_tensors)])
            t_c = time.perf_counter()
            for l in range(L):
                for t in range(w.n_tensors):
                    checkers.oracle_unpack(host_dst[l][t], outs[t], blobs[l][t])
        else:
            # the transposing pack: the oracle's HND <-> NHD permutation, block by block and
            # row by row, over the pages the ranges name
            heads, ntpb, row = w.xform
            B = 2 * heads * ntpb * row
            ids = [np.concatenate([np.arange(r[k] // B, (r[k] + r[2]) // B) for r in outs[0]])
                   .astype(np.uint32) for k in (0, 1)]
            for l in range(L):
                blob = np.empty(len(ids[0]) * B, dtype=np.uint8)
                olib.kvto_pack_hnd_to_nhd(host_src[l][0].ctypes.data, ids[0].ctypes.data,
                                          len(ids[0]), heads, ntpb, row, blob.ctypes.data)
                blobs.append([blob])
            t_c = time.perf_counter()
            for l in range(L):
                olib.kvto_unpack_nhd_to_hnd(host_dst[l][0].ctypes.data, ids[1].ctypes.data,
                                            len(ids[1]), heads, ntpb, row,
                                            blobs[l][0].ctypes.data)
        t_d = time.perf_counter()
        return (t_b - t_a, t_c - t_b, t_d - t_c), outs, blobs

    reps = [cpu_pass() for _ in range(5)]
    times = sorted(r[0] for r in reps)
    parse_s, pack_s, unpack_s = times[2]
    outs, blobs = reps[-1][1], reps[-1][2]
    parity = True
    for l in range(L if not mixed else 0):   # (mixed: the packed buffers are per half)
        for t in range(w.n_tensors):
            off = l * stride + plan0.tensor_offset(t)
            parity &= bool(np.array_equal(gpu_packed[off:off + len(blobs[l][t])], blobs[l][t]))
    for l in range(L):
        for t in range(w.n_tensors):
            parity &= bool(np.array_equal(side.dst[l][t].cpu().numpy(), host_dst[l][t]))
    P_s = sum(int(o[:, 2].sum()) for o in outs) * L
    total_s = parse_s + pack_s + unpack_s
    out["parity_vs_oracle"] = parity
    out["cpu_baseline"] = {
        "value": round(4.0 * P_s / total_s / 1e9, 2), "unit": "GB/s", "cores": 1,
        "kind": "port",
        "sample": "%d of %d layers of the same batch (%d requests): ParseBlock+merge %.1f ms, "
                  "pack %.1f ms, unpack %.1f ms; median of 5" %
                  (L, w.n_layers, len(w.tasks), parse_s * 1e3, pack_s * 1e3, unpack_s * 1e3),
        "host_cores_available": os.cpu_count(),
    }
    # ParseBlock alone for the whole batch: the reference's own functions (compiled from its
    # sources into oracle/_ref where that was possible), the oracle, and the product
    pb = {}
    if checkers.ref() is not None and not w.xform:
        tt = []
        with stdout_to_stderr():
            for _ in range(5):
                a = time.perf_counter()
                rc, _outs = checkers.ref_parse(pid, s_info, d_info, valid, tps, tpr, cpu_tasks)
                tt.append(time.perf_counter() - a)
                assert rc == 0
        pb["reference_ms"] = round(sorted(tt)[2] * 1e3, 3)
    tt = []
    for _ in range(5):
        a = time.perf_counter()
        rc, _outs = checkers.oracle_parse(pid, s_info, d_info, valid, tps, tpr, cpu_tasks)
        tt.append(time.perf_counter() - a)
    pb["oracle_ms"] = round(sorted(tt)[2] * 1e3, 3)
    parser = kvt.Parser(pid, s_info, d_info, valid, tps, tpr)
    tt = []
    for _ in range(5):
        lst = kvt.BlockLists()
        a = time.perf_counter()
        for t in cpu_tasks:
            parser.parse(t.struct, lst)
        tt.append(time.perf_counter() - a)
        lst.close()
    pb["product_ms"] = round(sorted(tt)[2] * 1e3, 3)
    pb["note"] = "%d requests, median of 5, one thread; output copies included" % len(cpu_tasks)
    out["cpu_baseline"]["parse_block"] = pb

    # all host cores, threads striding over layers (not the reference's threading model)
    nthr = min(16, os.cpu_count() or 1, L)
    if nthr > 1 and w.xform is None and w.n_tensors == 1:
        ptrs = (C.c_void_p * L)(*[host_src[l][0].ctypes.data for l in range(L)])
        runs0 = np.ascontiguousarray(outs[0])
        tb = int(runs0[:, 2].sum())
        blob = np.empty(L * tb, dtype=np.uint8)
        tt = []
        for _ in range(3):
            a = time.perf_counter()
            olib.kvto_pack_layers(ptrs, L, runs0.ctypes.data, len(runs0), blob.ctypes.data, tb,
                                  nthr)
            tt.append(time.perf_counter() - a)
        out["cpu_baseline_threads"] = {"pack_gbps": round(2.0 * tb * L / sorted(tt)[1] / 1e9, 2),
                                       "cores": nthr}
    log("cpu baseline done, parity:", out.get("parity_vs_oracle"))
    del host_src, host_dst, gpu_packed


def leg_latency(c, out):
    """Per-request KV pack latency. Three figures, each the median over the batch's requests:
    * latency_p50_us: GPU time from the first pack launch of layer 0 to the completion of the
      last layer on the side stream, the request packed layer by layer through a session (HIP
      events on the streams involved);
    * latency_wall_p50_us: host wall clock around the whole request -- ParseBlock, plan (cold:
      built for this request), one gated launch per layer, until the transport's wait for the
      last layer returns;
    * latency_single_launch_p50_us: GPU time of ONE launch covering all layers of the request
      (second, warm launch)."""
    torch, np, kvt, lib, args, pipeline = c.torch, c.np, c.kvt, c.lib, c.args, c.pipeline
    wls, sides, infos, tasks, first = c.wls, c.sides, c.infos, c.tasks, c.first
    strides, packed, stream, sh, new_event = c.strides, c.packed, c.stream, c.sh, c.new_event
    w, side = wls[0], sides[0]
    sender = c.senders[0]
    single, gated, wall, tail, grouped, tail_inline = [], [], [], [], [], []
    fill = [torch.zeros(256 << 20, dtype=torch.uint8, device="cuda") for _ in range(2)]
    reqs = list(range(len(w.tasks)))
    if len(reqs) < 5:                  # a single-request configuration: the same request again
        reqs = reqs * 5
    a, b = new_event(), new_event()
    # A sender keeps one session per destination (stream, events, counters): it exists before
    # the first timed request, made with an untimed run of request 0.
    lists = sender.parse([tasks[0][reqs[0]]])
    plan = kvt.Plan(0, lists, w.capacities("src"), w.capacities("dst"), xform=w.xform,
                    chunk_bytes=args.chunk_bytes)
    sess = kvt.Session(plan, side.src_cache, packed[0], plan.layer_bytes)
    step = sess.begin_step()
    for l in range(w.n_layers):
        sess.save_layer(l, sh)
    sess.wait_layer(w.n_layers - 1, step)
    torch.cuda.synchronize()
    held = (plan, lists)               # the session names this plan until the next set_plan
    for r in reqs:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        lists = sender.parse([tasks[0][r]])
        plan = kvt.Plan(0, lists, w.capacities("src"), w.capacities("dst"), xform=w.xform,
                        chunk_bytes=args.chunk_bytes)
        sess.set_plan(plan, packed[0], plan.layer_bytes)
        step = sess.begin_step()
        lib.kvt_event_record(a, sh)
        for l in range(w.n_layers):
            sess.save_layer(l, sh)
        lib.kvt_event_record(b, sess.side_stream)
        sess.wait_layer(w.n_layers - 1, step)
        wall.append((time.perf_counter() - t0) * 1e6)
        lib.kvt_event_synchronize(b)
        gated.append(ev_ms(lib, a, b) * 1e3)
        held[0].close()                # everything of the previous request has run
        held[1].close()
        held = (plan, lists)
        # The same request behind a busy compute stream: a plain 256 MiB copy per layer stands
        # in for the forward pass, so every layer's hop hides behind the next layer's compute
        # and what a request waits for is the tail: last layer computed -> last layer packed.
        step = sess.begin_step()
        for l in range(w.n_layers):
            assert lib.kvt_copy_linear(fill[1].data_ptr(), fill[0].data_ptr(), fill[0].numel(), sh) == 0
            if l == w.n_layers - 1:
                lib.kvt_event_record(a, sh)
            sess.save_layer(l, sh)
        lib.kvt_event_record(b, sess.side_stream)
        sess.wait_layer(w.n_layers - 1, step)
        lib.kvt_event_synchronize(b)
        tail.append(ev_ms(lib, a, b) * 1e3)
        # ... and with the last layer packed on the compute stream itself (no hop)
        step = sess.begin_step()
        for l in range(w.n_layers):
            assert lib.kvt_copy_linear(fill[1].data_ptr(), fill[0].data_ptr(), fill[0].numel(), sh) == 0
            if l == w.n_layers - 1:
                lib.kvt_event_record(a, sh)
                sess.save_layers_inline(l, 1, sh)
                lib.kvt_event_record(b, sh)
            else:
                sess.save_layer(l, sh)
        sess.wait_layer(w.n_layers - 1, step)
        lib.kvt_event_synchronize(b)
        tail_inline.append(ev_ms(lib, a, b) * 1e3)
        # the gated sequence again with one hop per group of four layers
        step = sess.begin_step()
        lib.kvt_event_record(a, sh)
        for l in range(0, w.n_layers, 4):
            sess.save_layers(l, min(4, w.n_layers - l), sh)
        lib.kvt_event_record(b, sess.side_stream)
        sess.wait_layer(w.n_layers - 1, step)
        lib.kvt_event_synchronize(b)
        grouped.append(ev_ms(lib, a, b) * 1e3)
        for rep in range(2):   # second run is the measurement
            lib.kvt_event_record(a, sh)
            plan.pack(side.src_cache, 0, w.n_layers, packed[0], plan.layer_bytes, sh)
            lib.kvt_event_record(b, sh)
        lib.kvt_event_synchronize(b)
        single.append(ev_ms(lib, a, b) * 1e3)
    torch.cuda.synchronize()
    sess.close()
    c.keep_objs.append(held)
    # The same per-layer sequence as ONE captured graph over a plan slot: per request ParseBlock,
    # refill of the slot, launch of the graph, until the transport's wait for the last layer
    # returns (host clock); and GPU time of the replay alone.
    if args.plan == "ranges":
        caps = (w.capacities("src"), w.capacities("dst"))
        chunk = plan_chunk_bytes(kvt, first[0][1], caps, w.xform, args.chunk_bytes)
        plan0 = first[0][0]
        slot = kvt.PlanSlot(0, w.n_tensors, caps[0], caps[1], max_entries=max(1, plan0.num_chunks),
                            xform=w.xform, chunk_bytes=chunk, max_layer_bytes=strides[0])
        gsess = kvt.Session(slot, side.src_cache, packed[0], strides[0])
        gs = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(gs):
            with torch.cuda.graph(graph, stream=gs):
                for l in range(w.n_layers):
                    gsess.save_layer(l, gs.cuda_stream)
                gsess.join(gs.cuda_stream)
        g_wall, g_gpu, g_parse = [], [], []
        with torch.cuda.stream(gs):
            for r in [reqs[0]] + reqs:           # the first pass warms up
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                lists = sender.parse([tasks[0][r]])
                t1 = time.perf_counter()
                slot.fill(lists, gs.cuda_stream)
                step = gsess.begin_step()
                lib.kvt_event_record(a, gs.cuda_stream)
                graph.replay()
                lib.kvt_event_record(b, gs.cuda_stream)
                gsess.wait_layer(w.n_layers - 1, step)
                g_wall.append((time.perf_counter() - t0) * 1e6)
                g_parse.append((t1 - t0) * 1e6)
                lib.kvt_event_synchronize(b)
                g_gpu.append(ev_ms(lib, a, b) * 1e3)
                lists.close()
        torch.cuda.synchronize()
        # what the replay costs when there is nothing to move: the same graph over an empty batch
        # (2 kernel nodes per layer -- the pack, which ends at once, and the signal -- chained
        # through the side stream): the price of per-layer launches and signals in a graph
        empty = kvt.BlockLists()
        g_floor = []
        with torch.cuda.stream(gs):
            slot.fill(empty, gs.cuda_stream)
            for rep in range(6):
                step = gsess.begin_step()
                lib.kvt_event_record(a, gs.cuda_stream)
                graph.replay()
                lib.kvt_event_record(b, gs.cuda_stream)
                gsess.wait_layer(w.n_layers - 1, step)
                lib.kvt_event_synchronize(b)
                g_floor.append(ev_ms(lib, a, b) * 1e3)
        empty.close()
        out["latency_graph_replay_empty_batch_gpu_p50_us"] = round(statistics.median(g_floor[1:]), 2)
        # the last request once more through a plan of its own: same bytes
        with torch.cuda.stream(gs):
            lists = sender.parse([tasks[0][reqs[-1]]])
            slot.fill(lists, gs.cuda_stream)
            gsess.begin_step()
            graph.replay()
        lists.close()
        torch.cuda.synchronize()
        lists = sender.parse([tasks[0][reqs[-1]]])
        fresh = kvt.Plan(0, lists, caps[0], caps[1], xform=w.xform, chunk_bytes=chunk)
        probe = torch.empty(max(1, strides[0]), dtype=torch.uint8, device="cuda")
        fresh.pack(side.src_cache, w.n_layers - 1, 1, probe, strides[0], gs.cuda_stream)
        gs.synchronize()
        nb = fresh.layer_bytes
        off = (w.n_layers - 1) * strides[0]
        out["latency_graph_replay_equals_fresh_plan"] = bool(torch.equal(probe[:nb], packed[0][off:off + nb]))
        out["latency_graph_replay_p50_us"] = round(statistics.median(g_wall[1:]), 2)
        out["latency_graph_replay_gpu_p50_us"] = round(statistics.median(g_gpu[1:]), 2)
        out["latency_graph_replay_parse_p50_us"] = round(statistics.median(g_parse[1:]), 2)
        gsess.close()
        fresh.close()
        lists.close()
        slot.close()
        del graph, probe
    out["latency_p50_us"] = round(statistics.median(gated), 2)
    out["latency_wall_p50_us"] = round(statistics.median(wall), 2)
    out["latency_groups_of_4_layers_p50_us"] = round(statistics.median(grouped), 2)
    out["latency_single_launch_p50_us"] = round(statistics.median(single), 2)
    out["latency_after_last_layer_p50_us"] = round(statistics.median(tail), 2)
    out["latency_after_last_layer_inline_p50_us"] = round(statistics.median(tail_inline), 2)
    del fill
    out["latency_note"] = ("per request (%d timed): latency_p50_us = GPU time from the first "
                           "pack launch of layer 0 to the completion of layer %d on the side "
                           "stream, one event-gated launch per layer "
                           "(latency_groups_of_4_layers_p50_us: per four layers, "
                           "kvt_session_save_layers); latency_wall_p50_us = host "
                           "clock from before ParseBlock (plan built cold) until the wait for the "
                           "last layer returns; latency_single_launch_p50_us = one warm launch "
                           "covering all layers; latency_after_last_layer_p50_us = the gated "
                           "sequence behind a busy compute stream (a 256 MiB copy per layer as "
                           "the forward pass): GPU time from the end of the last layer's compute "
                           "to the completion of its pack "
                           "(latency_after_last_layer_inline_p50_us: the last layer packed on "
                           "the compute stream itself, kvt_session_save_layers_inline); "
                           "latency_graph_replay_p50_us = the per-layer sequence captured once "
                           "into a hipGraph over a plan slot, host clock per request from before "
                           "ParseBlock (latency_graph_replay_parse_p50_us of it) through "
                           "kvt_plan_slot_fill and the launch of the graph until the wait for the "
                           "last layer returns (latency_graph_replay_gpu_p50_us: GPU time of the "
                           "replay between two events; latency_graph_replay_empty_batch_gpu_p50_us: "
                           "the same replay over an empty batch, i.e. what the launches and "
                           "signals of the layers cost by themselves)"
                           % (len(reqs), w.n_layers - 1))


def leg_session(c, out):
    """Layer-by-layer packing through an event-gated session, eager and replayed from a hipGraph."""
    torch, np, kvt, lib, args, pipeline = c.torch, c.np, c.kvt, c.lib, c.args, c.pipeline
    wls, sides, infos, tasks, first = c.wls, c.sides, c.infos, c.tasks, c.first
    strides, packed, stream, sh, new_event = c.strides, c.packed, c.stream, c.sh, c.new_event
    w, side = wls[0], sides[0]
    # layer-by-layer operation (the serving pattern: every layer is packed as soon as the
    # forward pass has produced it): one event-gated launch per layer on the side stream
    plan0 = first[0][0]
    sess = kvt.Session(plan0, side.src_cache, packed[0], strides[0])
    a, b = new_event(), new_event()
    for rep in range(2):
        lib.kvt_event_record(a, sh)
        for l in range(w.n_layers):
            sess.save_layer(l, sh)
        sess.join(sh)
        lib.kvt_event_record(b, sh)
    lib.kvt_event_synchronize(b)
    ms = ev_ms(lib, a, b)
    pay0 = sum(plan0.tensor_bytes(t) for t in range(w.n_tensors)) * w.n_layers
    out["per_layer_session"] = {"pack_ms_all_layers": round(ms, 4),
                                "pack_gbps": round(2.0 * pay0 / (ms * 1e-3) / 1e9, 1),
                                "launches": w.n_layers}
    # the same sequence captured once into a hipGraph and replayed
    gs = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(gs):
        with torch.cuda.graph(graph, stream=gs):
            for l in range(w.n_layers):
                sess.save_layer(l, gs.cuda_stream)
            sess.join(gs.cuda_stream)
    for rep in range(2):
        torch.cuda.synchronize()
        t_a = time.perf_counter()
        for _ in range(5):
            sess.begin_step()
            graph.replay()
        torch.cuda.synchronize()
        g_ms = (time.perf_counter() - t_a) / 5 * 1e3
    out["per_layer_session"]["graph_replay_ms_all_layers"] = round(g_ms, 4)
    # the transport's view of one replay: host time from the launch until wait_layer(l) returns,
    # for the first and the last layer (no stream or device synchronisation involved)
    torch.cuda.synchronize()
    step = sess.begin_step()
    t_a = time.perf_counter()
    graph.replay()
    sess.wait_layer(0, step)
    t_first = time.perf_counter()
    sess.wait_layer(w.n_layers - 1, step)
    t_last = time.perf_counter()
    out["per_layer_session"]["graph_replay_first_layer_signal_ms"] = round((t_first - t_a) * 1e3, 4)
    out["per_layer_session"]["graph_replay_last_layer_signal_ms"] = round((t_last - t_a) * 1e3, 4)
    torch.cuda.synchronize()
    del graph
    sess.close()
    if args.config == 2 and args.plan == "ranges":
        session_new_batches(c, out, g_ms)


def plan_chunk_bytes(kvt, lists, caps, xform, chunk_bytes):
    """The table-entry size kvt_plan_create picks for these lists (read off a host-only plan)."""
    probe = kvt.Plan(-1, lists, caps[0], caps[1], xform=xform, chunk_bytes=chunk_bytes)
    chunk = probe.host_tables()[2]
    probe.close()
    return chunk


def session_new_batches(c, out, frozen_ms):
    """The per-layer sequence captured ONCE over a plan slot and replayed with a NEW batch every
    time (kvt_plan_slot_fill before each launch of the graph): three batches on the same pools
    with different lengths and block tables in turn, ParseBlock + merge + refill inside the
    loop, the host running ahead of the GPU the way the timed steps do."""
    torch, kvt, lib, args, pipeline = c.torch, c.kvt, c.lib, c.args, c.pipeline
    w, side = c.wls[0], c.sides[0]
    caps = (w.capacities("src"), w.capacities("dst"))
    variants = [w] + [build_workload(2, args.scale, v)[0] for v in (1, 2)]
    v_tasks = [v.task_bufs() for v in variants]
    v_lists = [c.senders[0].parse(t) for t in v_tasks]
    chunk = plan_chunk_bytes(kvt, v_lists[0], caps, None, args.chunk_bytes)
    probes = [kvt.Plan(-1, l, caps[0], caps[1], chunk_bytes=chunk) for l in v_lists]
    entries = max(p.num_chunks for p in probes)
    room = max(p.layer_bytes for p in probes)
    payloads = [p.tensor_bytes(0) * w.n_layers for p in probes]
    for p in probes:
        p.close()
    slot = kvt.PlanSlot(0, 1, caps[0], caps[1], max_entries=entries, chunk_bytes=chunk,
                        max_layer_bytes=room)
    buf = torch.empty(room * w.n_layers, dtype=torch.uint8, device="cuda")
    sess = kvt.Session(slot, side.src_cache, buf, room)
    gs = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    slot.fill(v_lists[0], gs.cuda_stream)
    with torch.cuda.stream(gs):
        with torch.cuda.graph(graph, stream=gs):
            for l in range(w.n_layers):
                sess.save_layer(l, gs.cuda_stream)
            sess.join(gs.cuda_stream)
    res = {}
    with torch.cuda.stream(gs):
        for rep in range(2):           # the same batch again and again: the kernels' share
            torch.cuda.synchronize()
            t_a = time.perf_counter()
            for _ in range(5):
                sess.begin_step()
                graph.replay()
            torch.cuda.synchronize()
            res["graph_replay_slot_same_batch_ms"] = round((time.perf_counter() - t_a) / 5 * 1e3, 4)
        host = []
        e_a, e_b = c.new_event(), c.new_event()
        for rep in range(2):
            torch.cuda.synchronize()
            n = 6
            for i in range(n + 1):
                # steady state: the clock starts behind the first replay, whose batch the host
                # prepared with the GPU idle; from then on the host works while the GPU replays
                h0 = time.perf_counter()
                k = i % len(variants)
                lists = c.senders[0].parse(v_tasks[k])
                slot.fill(lists, gs.cuda_stream)
                lists.close()
                host.append(time.perf_counter() - h0)
                sess.begin_step()
                graph.replay()
                if i == 0:
                    lib.kvt_event_record(e_a, gs.cuda_stream)
            lib.kvt_event_record(e_b, gs.cuda_stream)
            lib.kvt_event_synchronize(e_b)
            new_ms = ev_ms(lib, e_a, e_b) / n
        last = n % len(variants)
    # what the last replay packed against a plan made for that batch alone (first and last layer)
    fresh = kvt.Plan(0, v_lists[last], caps[0], caps[1], chunk_bytes=chunk)
    ref = torch.empty(room, dtype=torch.uint8, device="cuda")
    same = True
    for l in (0, w.n_layers - 1):
        fresh.pack(side.src_cache, l, 1, ref, room, gs.cuda_stream)
        gs.synchronize()
        nb = fresh.tensor_bytes(0)
        same &= bool(torch.equal(ref[:nb], buf[l * room:l * room + nb]))
    mean_pay = sum(payloads[i % len(variants)] for i in range(1, n + 1)) / n
    res.update({
        "graph_replay_new_batch_ms": round(new_ms, 4),
        "graph_replay_new_batch_gbps": round(2.0 * mean_pay / (new_ms * 1e-3) / 1e9, 1),
        # (the fastest: a fill that finds the staging copy of two fills ago still unread waits
        # for the GPU, which is the back-pressure that keeps the host at most two steps ahead)
        "graph_replay_new_batch_host_ms": round(min(host) * 1e3, 4),
        "graph_replay_new_batch_vs_frozen_plan": round(
            (new_ms / mean_pay) / (frozen_ms / payloads[0]), 4),
        "graph_replay_new_batch_equals_fresh_plan": same,
        "graph_replay_new_batch_note":
            "one graph captured over a plan slot (%d entries of %d KiB), %d replays, each after "
            "ParseBlock + merge + kvt_plan_slot_fill of another batch (payloads %s MiB per "
            "launch of all layers), the host preparing the next batch while the GPU replays "
            "(HIP events from behind the first replay to behind the last); vs_frozen_plan = "
            "time per payload byte against graph_replay_ms_all_layers" %
            (entries, chunk >> 10, n, [round(p / 2**20) for p in payloads])})
    out["per_layer_session"].update(res)
    sess.close()
    fresh.close()
    slot.close()
    for l in v_lists:
        l.close()
    del buf, ref, graph


def leg_cu_usage(c, out):
    """Pack and unpack of the same batch with the copy launches limited to a share of the CUs
    (the reference's BLLM_KVTRANS_KERNEL_COPY_SM_USAGE): what a transfer that overlaps a
    forward pass gives up for leaving the rest of the device alone."""
    kvt, lib, sh, new_event = c.kvt, c.lib, c.sh, c.new_event
    w, side, plan0 = c.wls[0], c.sides[0], c.first[0][0]
    pay0 = sum(plan0.tensor_bytes(t) for t in range(w.n_tensors)) * w.n_layers
    rows = []
    try:
        for usage in (1.0, 0.5, 0.25, 0.125, 0.0625) if c.headline else (1.0, 0.5, 0.125):
            kvt.set_copy_cu_usage(0, usage)
            e = [new_event() for _ in range(3)]
            for rep in range(2):   # second run is the measurement
                lib.kvt_event_record(e[0], sh)
                plan0.pack(side.src_cache, 0, w.n_layers, c.packed[0], c.strides[0], sh)
                lib.kvt_event_record(e[1], sh)
                plan0.unpack(side.dst_cache, 0, w.n_layers, c.packed[0], c.strides[0], sh)
                lib.kvt_event_record(e[2], sh)
            lib.kvt_event_synchronize(e[2])
            rows.append({"usage": usage, "workgroups": kvt.get_copy_cu_usage(0)[1] or "one per slice",
                         "pack_gbps": round(2.0 * pay0 / (ev_ms(lib, e[0], e[1]) * 1e-3) / 1e9, 1),
                         "unpack_gbps": round(2.0 * pay0 / (ev_ms(lib, e[1], e[2]) * 1e-3) / 1e9, 1)})
    finally:
        kvt.set_copy_cu_usage(0, 1.0)
    out["cu_usage"] = rows


def leg_small_launch(c, out):
    """A launch small enough for the 256 MiB memory-side cache (config 1: 64 MiB) under the four
    load / store policies of kvt_set_copy_cached_load_max / kvt_set_copy_cached_store_max,
    against plain copies of the same size. Event intervals per launch, launches back to back on
    one stream. cold: 24 different requests of that size one after the other (1.5 GiB of blobs,
    so nothing a launch reads or writes is left in a cache from the launch before); pack_then_
    unpack: a request's unpack right behind its pack, requests cycling."""
    torch, kvt, lib, sh, new_event, pipeline = c.torch, c.kvt, c.lib, c.sh, c.new_event, c.pipeline
    from kvt_amd import workloads as W
    w, side = c.wls[0], c.sides[0]
    reps = 24
    ws = [W.llama8b_single(seed=20251 + 7 * r) for r in range(reps)]
    plans = [pipeline.build_plan(x, 0) for x in ws]
    stride = plans[0][0].layer_bytes
    nbytes = stride * w.n_layers
    blobs = [torch.empty(nbytes, dtype=torch.uint8, device="cuda") for _ in range(reps)]
    evs = [new_event() for _ in range(2 * reps + 1)]

    def timed(fns):
        for _ in range(3):              # the last pass is the measurement
            lib.kvt_event_record(evs[0], sh)
            for i, f in enumerate(fns):
                f()
                lib.kvt_event_record(evs[i + 1], sh)
            lib.kvt_event_synchronize(evs[len(fns)])
        return [ev_ms(lib, evs[i], evs[i + 1]) * 1e3 for i in range(len(fns))]

    def pk(r):
        return lambda: plans[r][0].pack(side.src_cache, 0, w.n_layers, blobs[r], stride, sh)

    def un(r):
        return lambda: plans[r][0].unpack(side.dst_cache, 0, w.n_layers, blobs[r], stride, sh)

    rows = []
    try:
        for loads, stores in ((0, 0), (0, 1), (1, 0), (1, 1)):
            lib.kvt_set_copy_cached_load_max(loads << 30)
            lib.kvt_set_copy_cached_store_max(stores << 30)
            cold_pack = statistics.median(timed([pk(r) for r in range(reps)]))
            cold_unpack = statistics.median(timed([un(r) for r in range(reps)]))
            seq = timed([f for r in range(reps // 2) for f in (pk(r), un(r))])
            rows.append({"loads": "plain" if loads else "nt", "stores": "plain" if stores else "sc0 sc1 nt",
                         "cold_pack_us": round(cold_pack, 2), "cold_unpack_us": round(cold_unpack, 2),
                         "pack_then_unpack_us": [round(statistics.median(seq[0::2]), 2),
                                                 round(statistics.median(seq[1::2]), 2)]})
    finally:
        lib.kvt_set_copy_cached_load_max(0)
        lib.kvt_set_copy_cached_store_max(0)
    res = {"policies": rows, "bytes_per_launch": nbytes}
    others = [torch.empty(nbytes, dtype=torch.uint8, device="cuda") for _ in range(reps)]
    for fn_name in ("kvt_copy_linear", "kvt_copy_runtime_d2d"):
        fn = getattr(lib, fn_name)
        t = timed([(lambda i=i: fn(others[i].data_ptr(), blobs[i].data_ptr(), nbytes, sh)) for i in range(reps)])
        res[fn_name + "_cold_us"] = round(statistics.median(t), 2)
    res["note"] = ("us per launch by event interval (launch gap included); the library's default is "
                   "the first row; the two copies are the cold ceilings for a launch of this size")
    for pl, ls in plans:
        pl.close()
        ls.close()
    out["small_launch"] = res


def leg_copy_ceilings(c, out):
    """Plain copies of the sizes the launches here have, by this library's linear copy kernel
    and by the runtime's own device-to-device hipMemcpyAsync: what the part gives a copy that
    gathers and scatters nothing. Each buffer pair is used once per measurement round, larger
    than the 256 MiB memory-side cache in total, so repeated rounds do not read from it."""
    torch, lib, sh, new_event = c.torch, c.lib, c.sh, c.new_event
    res = {}
    for name, n, pairs, rounds in (("64MiB", 64 << 20, 8, 6), ("4GiB", 4 << 30, 1, 4)):
        src = [torch.full((n,), 3, dtype=torch.uint8, device="cuda") for _ in range(pairs)]
        dst = [torch.empty(n, dtype=torch.uint8, device="cuda") for _ in range(pairs)]
        for fn_name in ("kvt_copy_linear", "kvt_copy_runtime_d2d"):
            fn = getattr(lib, fn_name)
            a, b = new_event(), new_event()
            times = []
            for rnd in range(rounds):
                lib.kvt_event_record(a, sh)
                for i in range(pairs):
                    assert fn(dst[i].data_ptr(), src[i].data_ptr(), n, sh) == 0, lib.kvt_last_error()
                lib.kvt_event_record(b, sh)
                lib.kvt_event_synchronize(b)
                times.append(ev_ms(lib, a, b) / pairs)
            t = statistics.median(times[1:])
            res["%s_%s" % (fn_name, name)] = {"us": round(t * 1e3, 2),
                                              "gbps": round(2.0 * n / (t * 1e-3) / 1e9, 1)}
        assert torch.equal(src[0], dst[0])
        del src, dst
    res["note"] = ("GB/s = bytes read + bytes written; back-to-back launches on one stream, "
                   "median of the rounds after the first")
    out["copy_ceilings"] = res


def leg_launchers(c, out):
    """The reference-shaped entry points on the same ranges."""
    torch, np, kvt, lib, args, pipeline = c.torch, c.np, c.kvt, c.lib, c.args, c.pipeline
    wls, sides, infos, tasks, first = c.wls, c.sides, c.infos, c.tasks, c.first
    strides, packed, stream, sh, new_event = c.strides, c.packed, c.stream, c.sh, c.new_event
    w, side = wls[0], sides[0]
    # the reference-shaped launchers (one launch per layer, ranges as three int64 arrays
    # resident on the device) and the converting bf16 -> fp8 gather
    if w.xform is None and args.plan == "ranges" and w.elem_dtype == "bf16":
        runs0 = first[0][1].tensor(0).astype(np.int64)
        so = torch.from_numpy(np.ascontiguousarray(runs0[:, 0])).cuda()
        ln = torch.from_numpy(np.ascontiguousarray(runs0[:, 2])).cuda()
        do = torch.from_numpy(np.concatenate([[0], np.cumsum(runs0[:, 2])[:-1]])).cuda()
        ln_e = ln // 2
        do_e = do // 2
        nb = int(runs0[:, 2].sum())
        a, b = new_event(), new_event()
        res = {}
        for name, fn, offs, lens, moved in (
                ("launch_copy_d2h_direct", lib.kvt_launch_copy_d2h_direct, do, ln, 2 * nb),
                ("launch_copy_d2h_bf16_to_fp8", lib.kvt_launch_copy_d2h_bf16_to_fp8, do_e,
                 ln_e, nb + nb // 2)):
            for rep in range(2):
                lib.kvt_event_record(a, sh)
                for l in range(w.n_layers):
                    rc = fn(side.src[l][0].data_ptr(), packed[0].data_ptr() + l * strides[0],
                            so.data_ptr(), offs.data_ptr(), lens.data_ptr(), len(runs0), 0, 0,
                            sh)
                    assert rc == 0, lib.kvt_last_error()
                lib.kvt_event_record(b, sh)
            lib.kvt_event_synchronize(b)
            res[name + "_gbps"] = round(moved * w.n_layers / (ev_ms(lib, a, b) * 1e-3) / 1e9, 1)
        res["note"] = ("%d launches of %d ranges each; GB/s = bytes read + bytes written; the "
                       "fp8 gather reads 2 bytes and writes 1 per element" %
                       (w.n_layers, len(runs0)))
        # the same launches limited to a share of the CUs (the reference's SM-usage knob)
        shares = []
        try:
            for usage in (0.5, 0.25, 0.125):
                kvt.set_copy_cu_usage(0, usage)
                row = {"usage": usage, "workgroups": kvt.get_copy_cu_usage(0)[1]}
                for name, fn, offs, lens, moved in (
                        ("launch_copy_d2h_direct", lib.kvt_launch_copy_d2h_direct, do, ln, 2 * nb),
                        ("launch_copy_d2h_bf16_to_fp8", lib.kvt_launch_copy_d2h_bf16_to_fp8, do_e,
                         ln_e, nb + nb // 2)):
                    for rep in range(2):
                        lib.kvt_event_record(a, sh)
                        for l in range(w.n_layers):
                            rc = fn(side.src[l][0].data_ptr(), packed[0].data_ptr() + l * strides[0],
                                    so.data_ptr(), offs.data_ptr(), lens.data_ptr(), len(runs0), 0, 0,
                                    sh)
                            assert rc == 0, lib.kvt_last_error()
                        lib.kvt_event_record(b, sh)
                    lib.kvt_event_synchronize(b)
                    row[name + "_gbps"] = round(moved * w.n_layers / (ev_ms(lib, a, b) * 1e-3) / 1e9, 1)
                shares.append(row)
        finally:
            kvt.set_copy_cu_usage(0, 1.0)
        res["cu_usage"] = shares
        # the reference's host entry point, called the way TCPChannel::send_data /
        # handle_kv_cache_data call it: pinned host buffer on the contiguous side, metadata
        # uploaded per call through the caller's two 8192-range buffers
        if nb <= (2 << 30):
            pin = torch.empty(nb, dtype=torch.uint8, pin_memory=True)
            meta_n = 3 * 8192
            dev_meta = torch.zeros(meta_n, dtype=torch.int64, device="cuda")
            host_meta = torch.zeros(meta_n, dtype=torch.int64).pin_memory()
            zeros = np.zeros(len(runs0), dtype=np.uint64)
            kb_send = np.ascontiguousarray(np.stack(
                [zeros, runs0[:, 0].astype(np.uint64), runs0[:, 2].astype(np.uint64)], axis=1))
            kb_recv = np.ascontiguousarray(first[0][1].tensor(0))
            Lh = min(4, w.n_layers)
            for name, direction, blocks, tensors in (
                    ("handle_data_d2h_pinned_gbps", 1, kb_send, side.src),
                    ("handle_data_h2d_pinned_gbps", 0, kb_recv, side.dst)):
                for rep in range(2):
                    torch.cuda.synchronize()
                    t_a = time.perf_counter()
                    for l in range(Lh):
                        rc = lib.kvt_copy_handle_data_with_kernel(
                            pin.data_ptr(), tensors[l][0].data_ptr(), blocks.ctypes.data,
                            len(blocks), nb, direction, 0, sh, dev_meta.data_ptr(),
                            host_meta.data_ptr(), 8192)
                        assert rc == 0, lib.kvt_last_error()
                        stream.synchronize()     # the reference syncs after every tensor
                    dt = time.perf_counter() - t_a
                res[name] = round(nb * Lh / dt / 1e9, 2)
            res["handle_data_note"] = ("%d layers, one call per layer incl. metadata upload and "
                                       "stream sync; GB/s = payload bytes over PCIe" % Lh)
        out["reference_shaped_launchers"] = res

    # pinned-host staging of packed layers, double buffered against the pack kernel


def leg_fp8_plan(c, out):
    """Configs 6 and 11 only (TP2 / TP8 -> TP1): the same batch with an fp8 receiver. The sender's plan
    converts bf16 to fp8 while it gathers (per-token arithmetic still in the kernel); checked
    against the oracle on the first layer."""
    torch, np, kvt, lib, args, pipeline = c.torch, c.np, c.kvt, c.lib, c.args, c.pipeline
    if args.config not in (6, 11) or args.plan != "runs":
        return
    import dataclasses
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import checkers
    w, side = c.wls[0], c.sides[0]
    d_info = dict(w.dst_info)
    d_info["token_sizes"] = [t // 2 for t in d_info["token_sizes"]]
    d_info["block_sizes"] = [b // 2 for b in d_info["block_sizes"]]
    w8 = dataclasses.replace(w, dst_info=d_info, notes=dict(w.notes, fp8=True),
                             name=w.name + ", fp8 receiver")
    t0 = time.perf_counter()
    plan, runs = pipeline.build_plan_runs(w8, 0, args.chunk_bytes)
    host_ms = (time.perf_counter() - t0) * 1e3
    dst_cache = kvt.Cache(0, side.dst, w8.capacities("dst"))      # the fp8 pool: half the bytes
    stride = plan.layer_bytes
    P8 = plan.tensor_bytes(0) * w8.n_layers                        # fp8 bytes on the wire
    packed = c.packed[0]
    assert packed.numel() >= stride * w8.n_layers
    a, b, d = c.new_event(), c.new_event(), c.new_event()
    pk, un = [], []
    for rep in range(4):
        lib.kvt_event_record(a, c.sh)
        plan.pack(side.src_cache, 0, w8.n_layers, packed, stride, c.sh)
        lib.kvt_event_record(b, c.sh)
        plan.unpack(dst_cache, 0, w8.n_layers, packed, stride, c.sh)
        lib.kvt_event_record(d, c.sh)
        lib.kvt_event_synchronize(d)
        if rep:
            pk.append(ev_ms(lib, a, b))
            un.append(ev_ms(lib, b, d))
    s_info, dd_info = w8.worker_infos()
    rc, valid, tps, tpr, pid, kind = checkers.oracle_select(w8.cache_shape, s_info, dd_info)
    rc2, outs = checkers.oracle_parse(pid, s_info, dd_info, valid, tps, tpr, w8.task_bufs(), fp8=True)
    assert rc == 0 and rc2 == 0
    ranges = np.ascontiguousarray(outs[0], dtype=np.uint64)
    layer0 = side.src[0][0].cpu().numpy()
    blob = np.zeros(int(ranges[:, 2].sum()), dtype=np.uint8)
    checkers.oracle().kvto_pack_bf16_to_fp8(layer0.ctypes.data, ranges.ctypes.data, len(ranges),
                                            blob.ctypes.data)
    parity = bool(np.array_equal(packed[:len(blob)].cpu().numpy(), blob))
    exp = np.zeros(w8.capacities("dst")[0], dtype=np.uint8)
    got = side.dst[0][0][:len(exp)].cpu().numpy()
    exp[:] = got
    checkers.oracle_unpack(exp, ranges, blob)      # idempotent on what the GPU already scattered
    parity &= bool(np.array_equal(got, exp))
    # the same two launches limited to a share of the device (pipelined persistent kernels)
    shares = []
    exp0 = np.zeros_like(exp)
    checkers.oracle_unpack(exp0, ranges, blob)
    try:
        for usage in (0.5, 0.25, 0.125):
            kvt.set_copy_cu_usage(0, usage)
            packed[:len(blob)].zero_()             # layer 0 of both sides: what the check reads
            side.dst[0][0][:len(exp)].zero_()
            torch.cuda.synchronize()
            for rep in range(2):   # second run is the measurement
                lib.kvt_event_record(a, c.sh)
                plan.pack(side.src_cache, 0, w8.n_layers, packed, stride, c.sh)
                lib.kvt_event_record(b, c.sh)
                plan.unpack(dst_cache, 0, w8.n_layers, packed, stride, c.sh)
                lib.kvt_event_record(d, c.sh)
                lib.kvt_event_synchronize(d)
            same = bool(np.array_equal(packed[:len(blob)].cpu().numpy(), blob)) and \
                bool(np.array_equal(side.dst[0][0][:len(exp)].cpu().numpy(), exp0))
            shares.append({"usage": usage, "workgroups": kvt.get_copy_cu_usage(0)[1],
                           "pack_gbps": round(3.0 * P8 / (ev_ms(lib, a, b) * 1e-3) / 1e9, 1),
                           "unpack_gbps": round(2.0 * P8 / (ev_ms(lib, b, d) * 1e-3) / 1e9, 1),
                           "parity_vs_oracle": same})
    finally:
        kvt.set_copy_cu_usage(0, 1.0)
    out["converting_plan"] = {
        "workload": w8.name, "fp8_payload_bytes": P8, "table_entries_per_layer": plan.num_chunks,
        "ranges_per_layer": int(len(ranges)), "host_parse_plan_ms": round(host_ms, 3),
        "pack_ms": round(statistics.mean(pk), 4), "unpack_ms": round(statistics.mean(un), 4),
        "pack_gbps": round(3.0 * P8 / (statistics.mean(pk) * 1e-3) / 1e9, 1),
        "unpack_gbps": round(2.0 * P8 / (statistics.mean(un) * 1e-3) / 1e9, 1),
        "parity_vs_oracle": parity, "cu_usage": shares,
        "note": "pack reads 2 bytes and writes 1 per element (bf16 -> fp8 E4M3), unpack moves "
                "the fp8 bytes; GB/s = bytes read + bytes written"}
    plan.close()
    runs.close()
    dst_cache.close()


def leg_frames(c, out):
    """Layer messages (TCP frame format) built around the GPU's output and consumed again:
    header + range metadata written by the host, blobs packed in HBM and placed by DMA;
    receiver parses the frame, DMAs the blobs back and unpacks."""
    torch, np, kvt, lib, args, pipeline = c.torch, c.np, c.kvt, c.lib, c.args, c.pipeline
    wls, sides, first = c.wls, c.sides, c.first
    from kvt_amd import binding
    w, side = wls[0], sides[0]
    if w.xform is not None or args.plan != "ranges":
        return
    plan, lists = first[0]
    lay = binding.wire_layout_of(binding.WIRE_TCP, lists)
    if lay.total_bytes > (3 << 30):
        return
    L = min(w.n_layers, 6)
    stg = kvt.Stager(0, lay.total_bytes, 2)
    dev = [torch.empty(plan.layer_bytes, dtype=torch.uint8, device="cuda") for _ in range(2)]
    ps = torch.cuda.Stream()
    cs = [torch.cuda.Stream(), torch.cuda.Stream()]     # a consumer stream per slot
    payload = sum(lay.blob_bytes[t] for t in range(w.n_tensors))
    host_write, host_parse, send_t, recv_t = [], [], [], []
    for phase in range(4):
        torch.cuda.synchronize()
        t_a = time.perf_counter()
        for l in range(L):
            slot = l % 2
            if l >= 2:
                stg.wait(slot)
            h0 = time.perf_counter()
            binding.wire_write_frame(binding.WIRE_TCP, stg.slot_ptr(slot), stg.slot_bytes, 1, l, lists)
            host_write.append(time.perf_counter() - h0)
            plan.pack(side.src_cache, l, 1, dev[slot], plan.layer_bytes, ps.cuda_stream)
            for t in range(w.n_tensors):
                stg.save_at(slot, lay.blob_offset[t], dev[slot].data_ptr() + plan.tensor_offset(t),
                            lay.blob_bytes[t], ps.cuda_stream)
        stg.wait(0)
        if L > 1:
            stg.wait(1)
        send_t.append(time.perf_counter() - t_a)
    # receiver: the last two frames are still in the slots; consume them repeatedly
    for phase in range(4):
        torch.cuda.synchronize()
        t_a = time.perf_counter()
        for l in range(L):
            slot = l % 2
            h0 = time.perf_counter()
            rc, reqid, layer, rlists, rlay = binding.wire_parse_frame(
                binding.WIRE_TCP, stg.slot_ptr(slot), lay.total_bytes, w.n_tensors)
            host_parse.append(time.perf_counter() - h0)
            assert rc == 0
            rlists.close()
            for t in range(w.n_tensors):
                stg.load_at(slot, rlay.blob_offset[t], dev[slot].data_ptr() + plan.tensor_offset(t),
                            rlay.blob_bytes[t], cs[slot].cuda_stream)
            plan.unpack(side.dst_cache, int(layer), 1, dev[slot], plan.layer_bytes, cs[slot].cuda_stream)
        cs[0].synchronize()
        cs[1].synchronize()
        recv_t.append(time.perf_counter() - t_a)
    out["layer_frames"] = {
        "frame_bytes": int(lay.total_bytes), "metadata_bytes": int(lay.total_bytes - payload),
        "send_gbps": round(L * payload / min(send_t[1:]) / 1e9, 2),
        "recv_gbps": round(L * payload / min(recv_t[1:]) / 1e9, 2),
        "host_write_frame_us": round(statistics.median(host_write) * 1e6, 1),
        "host_parse_frame_us": round(statistics.median(host_parse) * 1e6, 1),
        "note": "%d layer messages through 2 pinned slots; GB/s = payload over PCIe" % L}
    stg.close()


def leg_store_objects(c, out):
    """KVStore block objects (one per block and layer, or one per block over all layers):
    pack rate in HBM and save rate through the pinned stager."""
    torch, np, kvt, lib, args, pipeline = c.torch, c.np, c.kvt, c.lib, c.args, c.pipeline
    wls, sides, new_event, sh = c.wls, c.sides, c.new_event, c.sh
    w, side = wls[0], sides[0]
    from kvt_amd.ctypes_defs import SHAPE_FLASH
    if (w.cache_shape != SHAPE_FLASH or w.xform is not None or
            w.src_info["block_sizes"] != w.dst_info["block_sizes"]):
        return
    s_info, d_info = w.worker_infos()
    ids = sorted({b for t in w.tasks for b in t[3][0]})[:4096]
    rng = np.random.default_rng(1)
    dst_ids = rng.permutation(w.dst_info["layer_num_blocks"])[:len(ids)]
    lists, ob = kvt.block_object_lists(w.cache_shape, s_info, d_info, ids, dst_ids)
    L = w.n_layers
    res = {"blocks": len(ids), "object_bytes_per_layer": ob, "layers": L}
    for name, objects in (("per_block_and_layer", None), ("per_block_all_layers", (ob, L * ob))):
        plan = kvt.Plan(0, lists, w.capacities("src"), w.capacities("dst"), objects=objects)
        stride = ob if objects else plan.layer_bytes
        buf = torch.empty(len(ids) * ob * L, dtype=torch.uint8, device="cuda")
        a, b = new_event(), new_event()
        for rep in range(2):
            lib.kvt_event_record(a, sh)
            plan.pack(side.src_cache, 0, L, buf, stride, sh)
            lib.kvt_event_record(b, sh)
        lib.kvt_event_synchronize(b)
        res[name + "_pack_gbps"] = round(2.0 * len(ids) * ob * L / (ev_ms(lib, a, b) * 1e-3) / 1e9, 1)
        plan.close()
        del buf
    # save: per-layer object arrays through two pinned slots, several layers per transfer
    plan = kvt.Plan(0, lists, w.capacities("src"), w.capacities("dst"))
    lbytes = plan.layer_bytes
    group = max(1, min(L, -(-(256 << 20) // lbytes)))
    n_groups = max(1, min(6, L // group))
    stg = kvt.Stager(0, group * lbytes, 2)
    bufs = [torch.empty(group * lbytes, dtype=torch.uint8, device="cuda") for _ in range(2)]
    ps = torch.cuda.Stream()
    times = []
    for phase in range(3):
        torch.cuda.synchronize()
        t_a = time.perf_counter()
        for g in range(n_groups):
            slot = g % 2
            if g >= 2:
                stg.wait(slot)
            plan.pack(side.src_cache, g * group, group, bufs[slot], lbytes, ps.cuda_stream)
            stg.save(slot, bufs[slot], group * lbytes, ps.cuda_stream)
        stg.wait(0)
        if n_groups > 1:
            stg.wait(1)
        times.append(time.perf_counter() - t_a)
    res["save_gbps"] = round(n_groups * group * len(ids) * ob / min(times[1:]) / 1e9, 2)
    res["save_note"] = "%d transfers of %d layer(s) x %d objects" % (n_groups, group, len(ids))
    stg.close()
    plan.close()
    # the same objects (one per block, all layers) through the pinned ring keyed by block hash:
    # batches of 256 blocks, of which every fourth is stored already; then loaded back by hash
    nb = min(1024, len(ids))
    entry = ob * L
    ring = kvt.ObjectRing(0, entry, nb, 16)
    keys = [int(b).to_bytes(8, "little") + b"blockkey" for b in ids[:nb]]
    pre = list(range(0, nb, 4))
    e_pre, _ = ring.reserve([keys[i] for i in pre])
    ring.commit(e_pre)
    objs = torch.empty(256 * entry, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    t_a = time.perf_counter()
    saved = 0
    for first_blk in range(0, nb, 256):
        batch = list(range(first_blk, min(nb, first_blk + 256)))
        e, new = ring.reserve([keys[i] for i in batch])
        todo = [i for i, n in zip(batch, new) if n]
        lst, _ = kvt.block_object_lists(w.cache_shape, s_info, d_info, [ids[i] for i in todo],
                                        [dst_ids[i] for i in todo])
        pl = kvt.Plan(0, lst, w.capacities("src"), w.capacities("dst"), objects=(ob, entry))
        pl.pack(side.src_cache, 0, L, objs, ob, ps.cuda_stream)
        ring.save(e[new], objs.data_ptr(), entry, ps.cuda_stream)
        c.keep_objs.append((pl, lst))
        saved += len(todo)
    ps.synchronize()
    t_b = time.perf_counter()
    e, found = ring.lookup(keys)
    back = torch.empty(256 * entry, dtype=torch.uint8, device="cuda")
    hits = e[found]
    torch.cuda.synchronize()
    t_c = time.perf_counter()
    for first_blk in range(0, len(hits), 256):
        part = hits[first_blk:first_blk + 256]
        ring.load(part, back.data_ptr(), entry, ps.cuda_stream)
    ps.synchronize()
    t_d = time.perf_counter()
    res["hash_ring"] = {"entries": nb, "entry_bytes": entry, "blocks_saved": saved,
                        "blocks_skipped_as_stored": nb - saved,
                        "save_gbps": round(saved * entry / (t_b - t_a) / 1e9, 2),
                        "load_gbps": round(len(hits) * entry / (t_d - t_c) / 1e9, 2),
                        "note": "batches of 256 blocks: reserve by hash, pack the missing blocks "
                                "(all layers per object), DMA into the ring; load: the entries "
                                "found by hash, scattered ones by one kernel launch over PCIe, "
                                "long runs by DMA"}
    ring.close()
    out["kvstore_objects"] = res


def leg_staging(c, out):
    """Packed layers through pinned host memory, double buffered against the kernels."""
    torch, np, kvt, lib, args, pipeline = c.torch, c.np, c.kvt, c.lib, c.args, c.pipeline
    wls, sides, infos, tasks, first = c.wls, c.sides, c.infos, c.tasks, c.first
    strides, packed, stream, sh, new_event = c.strides, c.packed, c.stream, c.sh, c.new_event
    w, side = wls[0], sides[0]
    # Small layers are grouped so that one transfer is at least 256 MiB (a copy has a fixed
    # start-up cost of some tens of microseconds; config 1's layers are 2 MiB).
    plan = first[0][0]
    lbytes = plan.layer_bytes
    if 0 < lbytes < (3 << 30):
        group = max(1, min(w.n_layers, -(-(256 << 20) // lbytes)))
        n_groups = max(1, min(8, w.n_layers // group))
        nbytes = group * lbytes
        pay_group = sum(plan.tensor_bytes(t) for t in range(w.n_tensors)) * group
        ceil = {}
        for name, d in (("d2h", 1), ("h2d", 0)):
            r = C.c_double()
            assert lib.kvt_measure_pcie(0, d, min(nbytes, 1 << 30), 5, C.byref(r)) == 0
            ceil[name] = r.value
        stg = kvt.Stager(0, nbytes, 2)
        bufs = [torch.empty(nbytes, dtype=torch.uint8, device="cuda") for _ in range(2)]

        def save_pass(ps_, groups):
            torch.cuda.synchronize()
            a = time.perf_counter()
            for g in range(groups):
                slot = g % 2
                if g >= 2:
                    stg.wait(slot)
                plan.pack(side.src_cache, g * group, group, bufs[slot], lbytes, ps_.cuda_stream)
                stg.save(slot, bufs[slot], nbytes, ps_.cuda_stream)
            stg.wait(0)
            if groups > 1:
                stg.wait(1)
            return time.perf_counter() - a

        def load_pass(cs_, groups):
            torch.cuda.synchronize()
            a = time.perf_counter()
            for g in range(groups):
                # a consumer stream per slot: a load waits for what was queued on its consumer
                # stream, which then is the slot's last unpack and not the other slot's
                slot = g % 2
                stg.load(slot, bufs[slot], nbytes, cs_[slot].cuda_stream)
                plan.unpack(side.dst_cache, g * group, group, bufs[slot], lbytes, cs_[slot].cuda_stream)
            cs_[0].synchronize()
            cs_[1].synchronize()
            return time.perf_counter() - a

        # Which streams the caller uses matters: HIP maps streams onto a few hardware queues, and a
        # stream that waits (a consumer stream for its transfer, the copy stream for a pack)
        # parks that wait in its queue for as long as it takes; another stream mapped to the same
        # queue gets nothing through meanwhile, and what should overlap takes turns. Which
        # streams share a queue cannot be asked, only measured: four sets of producer / consumer
        # streams are tried with a short pass each and the best one is used (what a deployment
        # does once at start-up).
        probe_groups = min(n_groups, 4)
        sets = [(torch.cuda.Stream(), [torch.cuda.Stream(), torch.cuda.Stream()]) for _ in range(4)]
        one_way = []
        for st in sets:
            save_pass(st[0], min(2, probe_groups))
            t_s = save_pass(st[0], probe_groups)
            load_pass(st[1], min(2, probe_groups))
            t_l = load_pass(st[1], probe_groups)
            one_way.append(round(2 * pay_group * probe_groups / (t_s + t_l) / 1e9, 2))
        ps, cs = sets[max(range(4), key=lambda k: one_way[k])]
        d2h_t = [save_pass(ps, n_groups) for phase in range(4)]      # the first pass warms up
        h2d_t = [load_pass(cs, n_groups) for phase in range(4)]
        d2h_s, h2d_s = statistics.median(d2h_t[1:]), statistics.median(h2d_t[1:])
        pay = sum(plan.tensor_bytes(t) for t in range(w.n_tensors)) * group * n_groups
        # Both directions at once: a saving and a loading stager side by side, against two plain
        # pinned <-> device copies of the same size running concurrently on two streams.
        both = [C.c_double(), C.c_double()]
        assert lib.kvt_measure_pcie_both_ways(0, min(nbytes, 1 << 30), 5, C.byref(both[0]),
                                              C.byref(both[1])) == 0, lib.kvt_last_error()
        stg_in = kvt.Stager(0, nbytes, 2)
        bufs_in = [torch.empty(nbytes, dtype=torch.uint8, device="cuda") for _ in range(2)]
        for slot in range(2):           # what the loading side brings in: the groups saved last
            stg_in.slot_array(slot, nbytes)[:] = stg.slot_array(slot, nbytes)
        def both_ways(ps_, cs_, groups):
            """One pass with the given producer / consumer streams -> (save seconds, load seconds)."""
            torch.cuda.synchronize()
            a = time.perf_counter()
            for g in range(groups):
                slot = g % 2
                if g >= 2:
                    stg.wait(slot)
                plan.pack(side.src_cache, (g % n_groups) * group, group, bufs[slot], lbytes, ps_.cuda_stream)
                stg.save(slot, bufs[slot], nbytes, ps_.cuda_stream)
                stg_in.load(slot, bufs_in[slot], nbytes, cs_[slot].cuda_stream)
                plan.unpack(side.dst_cache, (g % n_groups) * group, group, bufs_in[slot], lbytes,
                            cs_[slot].cuda_stream)
            stg.wait(0)
            if groups > 1:
                stg.wait(1)
            t_save = time.perf_counter() - a
            cs_[0].synchronize()
            cs_[1].synchronize()
            return t_save, time.perf_counter() - a

        # (the same four sets of streams, tried with both stagers at work; at least four
        # transfers each way, the groups repeating, so that there is something to overlap)
        bi_groups = max(n_groups, 4)
        quick = []
        for st in sets:
            both_ways(st[0], st[1], 2)
            t_s, t_l = both_ways(st[0], st[1], 4)
            quick.append(round(2 * pay_group * 4 / (t_s + t_l) / 1e9, 2))
        ps_b, cs_b = sets[max(range(4), key=lambda k: quick[k])]
        bi_save, bi_load = [], []
        for phase in range(4):
            t_s, t_l = both_ways(ps_b, cs_b, bi_groups)
            bi_save.append(t_s)
            bi_load.append(t_l)
        bs, bl = (statistics.median(bi_save[1:]) * n_groups / bi_groups,
                  statistics.median(bi_load[1:]) * n_groups / bi_groups)
        stg_in.close()
        del bufs_in
        out["staging"] = {
            "save_gbps": round(pay / d2h_s / 1e9, 2), "load_gbps": round(pay / h2d_s / 1e9, 2),
            "pcie_d2h_gbps": round(ceil["d2h"] / 1e9, 2), "pcie_h2d_gbps": round(ceil["h2d"] / 1e9, 2),
            "save_frac_of_pcie": round(pay / d2h_s / ceil["d2h"], 4),
            "load_frac_of_pcie": round(pay / h2d_s / ceil["h2d"], 4),
            "bidir_save_gbps": round(pay / bs / 1e9, 2), "bidir_load_gbps": round(pay / bl / 1e9, 2),
            "bidir_pcie_d2h_gbps": round(both[0].value / 1e9, 2),
            "bidir_pcie_h2d_gbps": round(both[1].value / 1e9, 2),
            "bidir_save_frac_of_pcie": round(pay / bs / both[0].value, 4),
            "bidir_load_frac_of_pcie": round(pay / bl / both[1].value, 4),
            "stream_sets_gbps": one_way,
            "bidir_stream_sets_gbps": quick,
            "bidir_note": "a saving and a loading stager at the same time (pack -> D2H beside H2D "
                          "-> unpack), each direction's payload over the time until that direction "
                          "has finished; ceiling: two plain copies of one transfer's size running "
                          "concurrently on two streams (kvt_measure_pcie_both_ways); "
                          "stream_sets_gbps / bidir_stream_sets_gbps: mean rate per direction of a "
                          "short pass with each of four sets of producer / consumer streams, one "
                          "direction at a time / both at once (streams that share a hardware queue "
                          "take turns where they should overlap), the best set is the one measured",
            "sample": "%d transfers of %d layer(s) = %.1f MiB each through 2 pinned slots, "
                      "pack / unpack of the group in one launch; median of 3 passes" %
                      (n_groups, group, nbytes / 2**20),
        }
        stg.close()


# HBM bytes moved by ONE launch over all layers, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs
# of this file (each counter scaled by what it reads for the plain copy kernel of known size):
# profiles/*_hbm_traffic.md. Keyed by (config, plan); valid for scale 1 and the automatic
# chunk size, and only for the kernel source they were measured with: tests/test_bench_contract.py
# compares KERNELS_SHA256 with llumnix-kv_amd/csrc/kvt_kernels.hip and fails when the file has
# changed since, so a stale table cannot pass unnoticed.
KERNELS_SHA256 = "aa1123ba9e7332ed676cb512bcb5997d9402593a554fe0ea56256a9a1a5cd47c"
MEASURED_TRAFFIC = {
    (1, "ranges"): {"pack": 134268079, "unpack": 134278234},
    (2, "ranges"): {"pack": 71013152265, "unpack": 73358397596},
    (3, "ranges"): {"pack": 85983237339, "unpack": 85984011093},
    (4, "ranges"): {"pack": 22690361783, "unpack": 22690413793},
    (5, "ranges"): {"pack": 45141172606, "unpack": 45141395495},
    (9, "ranges"): {"pack": 45141104254, "unpack": 45141166035},
}


def measured_traffic(args, direction):
    if args.scale != 1.0 or args.chunk_bytes != 0:
        return None
    row = MEASURED_TRAFFIC.get((args.config, args.plan))
    return row[direction] if row else None


def run_config(args, headline):
    """One configuration: caches resident in HBM, the timed steps, the side legs. Returns the
    dictionary that becomes the JSON line (headline) or a row of its "configs" list, and frees
    everything it allocated."""
    import gc

    import numpy as np
    import torch

    import kvt_amd as kvt
    from kvt_amd import pipeline

    lib = kvt.lib()
    full_wls = build_workload(args.config, args.scale)
    t_init = time.time()
    full_sides = [DeviceSide(torch, kvt, w, 7 + i) for i, w in enumerate(full_wls)]
    torch.cuda.synchronize()
    log("config %d: caches resident in %.1fs" % (args.config, time.time() - t_init))
    mixed = args.config == 5 and not args.sequential
    if mixed:
        # halves A and B of every workload's requests, on the same caches; a step is
        # (pack A || unpack B) then (pack B || unpack A): every request still goes both ways
        import dataclasses
        wls, sides = [], []
        for half in (0, 1):
            for w, sd in zip(full_wls, full_sides):
                h = len(w.tasks) // 2
                part = w.tasks[:h] if half == 0 else w.tasks[h:]
                wls.append(dataclasses.replace(w, tasks=part, name=w.name + " [half %s]" % "AB"[half]))
                sides.append(sd)
        n_half = len(full_wls)
    else:
        wls, sides = full_wls, full_sides

    infos = [w.worker_infos() for w in wls]
    tasks = [w.task_bufs() for w in wls]

    # per destination, once: parser selection and compilation (refresh_dst_info in the reference)
    senders = [pipeline.Sender(w.cache_shape, infos[i][0], infos[i][1]) for i, w in enumerate(wls)]
    caps = [(w.capacities("src"), w.capacities("dst")) for w in wls]

    def prepare(i):
        """host part of a step for workload i: ParseBlock + merge + plan upload"""
        w = wls[i]
        if args.plan == "runs":
            runs = senders[i].parse_runs(tasks[i])
            return kvt.Plan(0, runs, caps[i][0], caps[i][1], chunk_bytes=args.chunk_bytes), runs
        lists = senders[i].parse(tasks[i])
        plan = kvt.Plan(0, lists, caps[i][0], caps[i][1], xform=w.xform,
                        chunk_bytes=args.chunk_bytes)
        return plan, lists

    first = [prepare(i) for i in range(len(wls))]
    strides = [p.layer_bytes for p, _ in first]
    payload = [sum(p.tensor_bytes(t) for t in range(w.n_tensors)) * w.n_layers
               for (p, _), w in zip(first, wls)]
    P = sum(payload)
    packed = [torch.empty(max(1, s * w.n_layers), dtype=torch.uint8, device="cuda")
              for s, w in zip(strides, wls)]
    log("payload per step: %.3f GiB, chunks per layer: %s" %
        (P / 2**30, [p.num_chunks for p, _ in first]))

    stream = torch.cuda.Stream()
    sh = stream.cuda_stream
    made_events = []

    def new_event():
        e = C.c_void_p()
        assert lib.kvt_event_create(C.byref(e)) == 0, lib.kvt_last_error()
        made_events.append(e)
        return e

    s2 = torch.cuda.Stream()
    sh2 = s2.cuda_stream

    def launch_mixed(plans, evs):
        def go(i, pack, stream_handle):
            plan = plans[i][0]
            fn = plan.pack if pack else plan.unpack
            fn(sides[i].src_cache if pack else sides[i].dst_cache, 0, wls[i].n_layers, packed[i],
               strides[i], stream_handle)
        A, B = range(0, n_half), range(n_half, 2 * n_half)
        lib.kvt_event_record(evs[0], sh)
        start = torch.cuda.Event()
        start.record(stream)
        s2.wait_event(start)
        for i in A:
            go(i, True, sh)            # pack A          | stream 1
        for i in B:
            go(i, False, sh2)          # unpack B        | stream 2 (B was packed by the previous step)
        a_packed, b_unpacked = torch.cuda.Event(), torch.cuda.Event()
        a_packed.record(stream)
        b_unpacked.record(s2)
        lib.kvt_event_record(evs[1], sh)
        stream.wait_event(b_unpacked)  # pack B overwrites what unpack B read
        s2.wait_event(a_packed)        # unpack A needs pack A
        for i in B:
            go(i, True, sh)
        for i in A:
            go(i, False, sh2)
        done2 = torch.cuda.Event()
        done2.record(s2)
        stream.wait_event(done2)
        lib.kvt_event_record(evs[2], sh)

    def launch(plans, evs):
        if mixed:
            return launch_mixed(plans, evs)
        lib.kvt_event_record(evs[0], sh)
        for i, (plan, _) in enumerate(plans):
            plan.pack(sides[i].src_cache, 0, wls[i].n_layers, packed[i], strides[i], sh)
        lib.kvt_event_record(evs[1], sh)
        for i, (plan, _) in enumerate(plans):
            plan.unpack(sides[i].dst_cache, 0, wls[i].n_layers, packed[i], strides[i], sh)
        lib.kvt_event_record(evs[2], sh)

    if mixed:   # the first mixed step unpacks half B: give it packed data
        for i in range(n_half, 2 * n_half):
            first[i][0].pack(sides[i].src_cache, 0, wls[i].n_layers, packed[i], strides[i], sh)
    keep = [first]
    plans = first
    if args.cu_usage < 1.0:
        kvt.set_copy_cu_usage(0, args.cu_usage)
    for _ in range(args.warmup):
        launch(plans, [new_event() for _ in range(3)])
        plans = [prepare(i) for i in range(len(wls))]
        keep.append(plans)
        if len(keep) > 3:
            for pl, ls in keep.pop(1):
                pl.close()
                ls.close()
    torch.cuda.synchronize()

    events, host_ms = [], []
    t0 = time.perf_counter()
    for k in range(args.steps):
        evs = [new_event() for _ in range(3)]
        events.append(evs)
        launch(plans, evs)
        # host side of the following step (ParseBlock + merge + plan upload) overlaps this
        # step's GPU work; every timed step pays for one such preparation
        h0 = time.perf_counter()
        plans = [prepare(i) for i in range(len(wls))]
        keep.append(plans)
        if len(keep) > 3:               # plans of finished steps go back to the library's pool
            for pl, ls in keep.pop(1):
                pl.close()
                ls.close()
        host_ms.append((time.perf_counter() - h0) * 1e3)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    kvt.set_copy_cu_usage(0, 1.0)
    ms_per_step = wall / args.steps * 1e3
    pack_ms = [ev_ms(lib, e[0], e[1]) for e in events]
    unpack_ms = [ev_ms(lib, e[1], e[2]) for e in events]
    pack_avg, unpack_avg = statistics.mean(pack_ms), statistics.mean(unpack_ms)
    value = 4.0 * P / (ms_per_step * 1e-3) / 1e9
    achieved = 2.0 * P / (pack_avg * 1e-3) / 1e9
    if mixed:   # the two event intervals are the two phases; both directions run in each
        pack_avg = unpack_avg = (pack_avg + unpack_avg) / 2
        achieved = 2.0 * P / (pack_avg * 1e-3) / 1e9
    log("pack %.3f ms  unpack %.3f ms  host %.3f ms/step  wall %.3f ms/step" %
        (pack_avg, unpack_avg, statistics.mean(host_ms), ms_per_step))

    # instantiation names as a profiler prints them: <pack, [words,] capped>
    if first[0][0].num_strided_chunks:
        kernel = "kvt::strided_chunks_kernel<true, false, false> (pack)"
    elif wls[0].xform:
        kernel = "kvt::xform_chunks_kernel<true, false> (pack)"
    elif first[0][0].num_chunks <= 64:
        kernel = "kvt::copy_chunks_small_kernel<true, 0> (pack)"
    else:
        kernel = "kvt::copy_chunks_kernel<true, 0> (pack)"
    limited = args.cu_usage < 1.0
    if limited:   # the persistent kernels run instead; the counter table is for the unlimited ones
        kernel = "the persistent (CU-share limited) counterpart of " + kernel
    out = {
        "metric": "pack+unpack GB/s (bytes read + bytes written per second, whole job)",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8",
        "data": "synthetic",
        "config": {"workload": "; ".join(w.name for w in wls), "baseline_config": args.config,
                   "scale": args.scale, "layers": [w.n_layers for w in wls],
                   "requests": [len(w.tasks) for w in wls], "payload_bytes_per_step": P,
                   "chunk_bytes": args.chunk_bytes or "auto", "plan": args.plan,
                   "cu_usage": args.cu_usage,
                   "table_entries_per_layer": [p.num_chunks for p, _ in first]},
        "frac_hbm_peak": round(value * 1e9 / HBM_PEAK, 4),
        "pack_ms": round(pack_avg, 4),
        "unpack_ms": round(unpack_avg, 4),
        "pack_gbps": round(achieved, 1),
        "unpack_gbps": round(2.0 * P / (unpack_avg * 1e-3) / 1e9, 1),
        "host_parse_plan_ms": round(statistics.mean(host_ms), 4),
        "mode": ("mixed: (pack A || unpack B) then (pack B || unpack A) on two streams; pack_ms = "
                 "unpack_ms = mean phase time") if mixed else "sequential: pack all, then unpack all",
        "roofline": {"bound": "hbm", "kernel": kernel,
                     "achieved": round(achieved, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved * 1e9 / HBM_PEAK, 4),
                     "algorithmic_bytes_per_launch": 2 * P,
                     "traffic": None if limited else measured_traffic(args, "pack"),
                     "traffic_unpack": None if limited else measured_traffic(args, "unpack")},
    }
    keep_objs = []
    c = types.SimpleNamespace(torch=torch, np=np, kvt=kvt, lib=lib, args=args, pipeline=pipeline,
                              wls=wls, sides=sides, full_wls=full_wls, full_sides=full_sides,
                              mixed=mixed, infos=infos, tasks=tasks, first=first, strides=strides,
                              packed=packed, stream=stream, sh=sh, new_event=new_event, keep=keep,
                              senders=senders, keep_objs=keep_objs, headline=headline)
    # The timed region is over: a failure in a side leg must not take the measured line with
    # it. It is reported in "errors" (and on stderr, with the traceback) and fails the run.
    legs = [] if args.skip_cpu else [leg_cpu]
    if not args.skip_extras:
        legs += [leg_latency, leg_staging, leg_cu_usage]
        if args.config == 1:
            legs += [leg_small_launch]
        if headline:
            legs += [leg_session, leg_copy_ceilings, leg_launchers, leg_fp8_plan,
                     leg_frames, leg_store_objects]
    if args.legs:   # a profiling run of chosen legs only
        want = {"leg_" + name for name in args.legs.split(",")}
        every = [leg_latency, leg_staging, leg_cu_usage, leg_small_launch, leg_session, leg_copy_ceilings,
                 leg_launchers, leg_fp8_plan, leg_frames, leg_store_objects]
        unknown = want - {leg.__name__ for leg in every}
        if unknown:
            raise SystemExit("bench.py: --legs knows %s" % ", ".join(l.__name__[4:] for l in every))
        legs = [leg for leg in every if leg.__name__ in want]
    errors = {}
    for leg in legs:
        try:
            leg(c, out)
        except Exception as e:          # noqa: BLE001 - reported, not swallowed
            import traceback
            traceback.print_exc(file=sys.stderr)
            errors[leg.__name__] = "%s: %s" % (type(e).__name__, e)
    if errors:
        out["errors"] = errors
    # give everything back before the next configuration builds its caches
    torch.cuda.synchronize()
    for batch in keep:
        for pl, ls in batch:
            pl.close()
            ls.close()
    for pl, ls in keep_objs:
        pl.close()
        ls.close()
    for sd in full_sides:
        sd.src_cache.close()
        sd.dst_cache.close()
    for sender in senders:
        sender.close()
    for e in made_events:
        lib.kvt_event_destroy(e)
    del c, keep, keep_objs, first, plans, packed, sides, full_sides, wls, full_wls, events
    gc.collect()
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", type=int, default=0,
                    help="0 (default): the headline configuration 2 as the JSON line, followed by "
                         "the other four baseline configurations and config 9 (config 5 in the "
                         "reference's uniform-page arrangement) as rows of its \"configs\" list; "
                         "1-5: that baseline configuration alone (1 = the CPU-runnable case, 2 = "
                         "the headline); 6-8, 11: TP-remapping batches; 9: config 5 with the "
                         "reference's uniform 2 MiB pages; 10: the same model TP2 -> TP1")
    ap.add_argument("--scale", type=float, default=1.0, help="shrink the workload (debugging)")
    ap.add_argument("--chunk-bytes", type=int, default=0)
    ap.add_argument("--plan", choices=["ranges", "runs"], default="ranges",
                    help="runs: ParseBlock in closed form (strided runs), the per-token offset "
                         "arithmetic done by the copy kernel")
    ap.add_argument("--sequential", action="store_true",
                    help="config 5 only: pack everything, then unpack everything, instead of the "
                         "mixed mode (half of the requests packing while the other half unpacks)")
    ap.add_argument("--cpu-layers", type=int, default=16,
                    help="layers in the CPU baseline sample (16 layers x 5 passes of config 2 are "
                         "about 10 s of single-thread CPU work)")
    ap.add_argument("--cu-usage", type=float, default=1.0,
                    help="limit the timed pack / unpack launches to this share of the device "
                         "(kvt_set_copy_cu_usage; the reference's BLLM_KVTRANS_KERNEL_COPY_SM_USAGE)")
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--skip-extras", action="store_true", help="no latency / staging legs")
    ap.add_argument("--legs", default="",
                    help="comma-separated side legs to run instead of the default set (for a "
                         "profile of one of them): latency, staging, cu_usage, small_launch, session, "
                         "copy_ceilings, launchers, fp8_plan, frames, store_objects")
    ap.add_argument("--calibrate-copy-gib", type=float, default=0.0,
                    help="only run the plain linear copy kernel on this many GiB (profiler "
                         "counter calibration: its HBM traffic is known, 1 read + 1 write)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        raise SystemExit("bench.py: this build measures ONE MI355X; the path has no inter-GPU "
                         "part, so --gpus N with N > 1 is not supported.")

    import torch

    import kvt_amd as kvt

    lib = kvt.lib()
    if kvt.device_count() < 1:
        raise SystemExit("bench.py: no usable MI355X (gfx950) device; there is no CPU fallback")

    if args.calibrate_copy_gib > 0:
        # plain copies of one size, `steps` launches each of this library's linear copy kernel
        # and of the runtime's own device-to-device copy: counter calibration (known traffic)
        # and, under a kernel trace, the two copy ceilings for a launch of that size
        n = int(args.calibrate_copy_gib * 2**30)
        a = torch.full((n,), 3, dtype=torch.uint8, device="cuda")
        b = torch.empty(n, dtype=torch.uint8, device="cuda")
        res = {"calibration": "plain copies", "bytes": n, "launches": args.steps}
        for fn_name in ("kvt_copy_linear", "kvt_copy_runtime_d2d"):
            fn = getattr(lib, fn_name)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                assert fn(b.data_ptr(), a.data_ptr(), n, None) == 0
            torch.cuda.synchronize()
            dt = (time.perf_counter() - t0) / args.steps
            assert torch.equal(a, b)
            res[fn_name + "_gbps_read_plus_write"] = round(2 * n / dt / 1e9, 1)
            b.zero_()
        print(json.dumps(res))
        return

    all_configs = args.config == 0
    if all_configs:
        args.config = 2
    out = run_config(args, headline=True)
    if all_configs:
        # the other baseline configurations, full size, one after the other on the same GPU:
        # the timed steps, parity against the oracle on a sample of layers, the request
        # latencies and the staging path
        rows = []
        for cfg in (1, 3, 4, 5, 9):
            sub = argparse.Namespace(**vars(args))
            sub.config, sub.plan, sub.chunk_bytes = cfg, "ranges", 0
            sub.cpu_layers = min(args.cpu_layers, 4)
            try:
                r = run_config(sub, headline=False)
            except Exception as e:      # noqa: BLE001 - reported, not swallowed
                import traceback
                traceback.print_exc(file=sys.stderr)
                out.setdefault("errors", {})["config %d" % cfg] = "%s: %s" % (type(e).__name__, e)
                continue
            row = {"config": cfg, "workload": r["config"]["workload"],
                   "payload_bytes_per_step": r["config"]["payload_bytes_per_step"]}
            for key in ("value", "ms_per_step", "pack_gbps", "unpack_gbps", "pack_ms", "unpack_ms",
                        "frac_hbm_peak", "host_parse_plan_ms", "mode", "parity_vs_oracle",
                        "latency_p50_us", "latency_wall_p50_us", "latency_single_launch_p50_us",
                        "latency_groups_of_4_layers_p50_us", "latency_graph_replay_p50_us",
                        "latency_graph_replay_gpu_p50_us", "latency_graph_replay_parse_p50_us",
                        "latency_graph_replay_equals_fresh_plan",
                        "latency_graph_replay_empty_batch_gpu_p50_us",
                        "latency_after_last_layer_p50_us", "latency_after_last_layer_inline_p50_us",
                        "cu_usage", "small_launch",
                        "staging", "roofline", "cpu_baseline", "errors"):
                if key in r:
                    row[key] = r[key]
            row["frac"] = r["roofline"]["frac"]
            rows.append(row)
            if "errors" in r:
                out.setdefault("errors", {})["config %d" % cfg] = r["errors"]
        out["configs"] = rows
    print(json.dumps(out), flush=True)
    if out.get("errors"):
        raise SystemExit(1)


if __name__ == "__main__":
    main()
