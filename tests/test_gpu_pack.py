"""GPU parity tests: the HIP pack / unpack path, called through the C ABI of
libkvt_hip.so, against the CPU oracle on identical seeded caches and block
tables. Bit-exact (byte work). Needs a real MI355X: run with `-m gpu`."""
import ctypes as C

import numpy as np
import pytest

import checkers
import kvt_amd
from kvt_amd import pipeline, workloads

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _dev_bytes(n, seed=None, dtype="bf16"):
    """n bytes of seeded cache content on the GPU (as a uint8 tensor)."""
    g = torch.Generator(device="cuda")
    g.manual_seed(0 if seed is None else seed)
    if dtype == "bf16":
        t = (torch.rand(n // 2, generator=g, device="cuda") * 2 - 1).to(torch.bfloat16)
        return t.view(torch.uint8)
    if dtype == "fp8":
        t = torch.randn(n, generator=g, device="cuda").clamp_(-448, 448).to(torch.float8_e4m3fn)
        return t.view(torch.uint8)
    if dtype == "f32":
        return torch.randn(n // 4, generator=g, device="cuda").view(torch.uint8)
    return torch.randint(0, 256, (n,), generator=g, device="cuda", dtype=torch.uint8)


def _host(t):
    return t.cpu().numpy()


def _make_caches(w, side, seed, dtype=None, fill=True):
    caps = w.capacities(side)
    layers = []
    for l in range(w.n_layers):
        row = []
        for t, cap in enumerate(caps):
            if fill:
                row.append(_dev_bytes(cap, seed * 1000 + l * 8 + t, dtype or w.elem_dtype))
            else:
                row.append(torch.full((cap,), 0xA5, dtype=torch.uint8, device="cuda"))
        layers.append(row)
    return layers


def _oracle_lists(w):
    """merged per-tensor range lists from the oracle (independent of the product parser)"""
    src, dst = w.worker_infos()
    rc, valid, tps, tpr, pid, kind = checkers.oracle_select(w.cache_shape, src, dst)
    assert rc == 0
    rc, outs = checkers.oracle_parse(pid, src, dst, valid, tps, tpr, w.task_bufs())
    assert rc == 0
    if kind == 0:
        outs = [checkers.oracle_merge(o)[0] for o in outs]
    return outs


def _check_pack_unpack(w, seed=1, chunk_bytes=0, layers_per_launch=None):
    plan, lists = pipeline.build_plan(w, 0, chunk_bytes)
    o_lists = _oracle_lists(w)
    for t in range(w.n_tensors):
        assert np.array_equal(lists.tensor(t), o_lists[t])
    src_layers = _make_caches(w, "src", seed)
    dst_layers = _make_caches(w, "dst", seed + 1, fill=False)
    src_cache = kvt_amd.Cache(0, src_layers, w.capacities("src"))
    dst_cache = kvt_amd.Cache(0, dst_layers, w.capacities("dst"))
    stride = plan.layer_bytes
    packed = torch.zeros(w.n_layers * stride, dtype=torch.uint8, device="cuda")
    step = layers_per_launch or w.n_layers
    for first in range(0, w.n_layers, step):
        n = min(step, w.n_layers - first)
        plan.pack(src_cache, first, n, packed.data_ptr() + first * stride, stride)
    torch.cuda.synchronize()
    packed_h = _host(packed)
    for l in range(w.n_layers):
        for t in range(w.n_tensors):
            blob = checkers.oracle_pack(_host(src_layers[l][t]), o_lists[t])
            off = l * stride + plan.tensor_offset(t)
            assert plan.tensor_bytes(t) == len(blob)
            assert np.array_equal(packed_h[off:off + len(blob)], blob), (l, t)
    for first in range(0, w.n_layers, step):
        n = min(step, w.n_layers - first)
        plan.unpack(dst_cache, first, n, packed.data_ptr() + first * stride, stride)
    torch.cuda.synchronize()
    for l in range(w.n_layers):
        for t in range(w.n_tensors):
            exp = np.full(w.capacities("dst")[t], 0xA5, dtype=np.uint8)
            off = l * stride + plan.tensor_offset(t)
            checkers.oracle_unpack(exp, o_lists[t], packed_h[off:off + plan.tensor_bytes(t)])
            assert np.array_equal(_host(dst_layers[l][t]), exp), (l, t)
    return plan


def test_config1_llama8b_single_request_full_size():
    w = workloads.llama8b_single()  # 32 layers x 64 MiB, 1 request x 512 tokens
    plan = _check_pack_unpack(w)
    assert plan.layer_bytes == 2 * 1024 * 1024
    assert plan.num_chunks == 64


@pytest.mark.parametrize("chunk", [0, 4096, 65536])
def test_config2_shape_reduced_pool(chunk):
    w = workloads.llama8b_batch(n_layers=3, src_pool=512, dst_pool=768, n_req=6, min_tok=100,
                                max_tok=1500)
    _check_pack_unpack(w, chunk_bytes=chunk, layers_per_launch=2)


def test_config3_plain_hnd_ranges():
    w = workloads.llama70b_flashinfer(n_layers=2, pool=256, n_req=3, tokens=600, transpose=False)
    _check_pack_unpack(w)


def test_config4_mla_and_indexer_two_tensors():
    w = workloads.deepseek_mla(n_layers=3, pool=64, n_req=3, tokens=1000)
    plan = _check_pack_unpack(w)
    assert plan.tensor_offset(1) % 256 == 0 and plan.tensor_offset(1) >= plan.tensor_bytes(0)


def test_config5_attention_pages_and_gdn_states():
    _check_pack_unpack(workloads.qwen3next_attn(n_layers=2, pool=512, n_req=5, tokens=700))
    _check_pack_unpack(workloads.qwen3next_gdn(n_layers=2, slots=12, n_req=5), chunk_bytes=65536)


def test_config5_reference_layout_uniform_pages_shared_by_attention_and_gdn():
    w = workloads.qwen3next_uniform_pages(n_layers=2, pool=40, n_req=5)
    lists = _oracle_lists(w)[0]
    assert len(lists) <= 5 * 7 and int(lists[:, 2].sum()) == 5 * 7 * (2 << 20)
    _check_pack_unpack(w)
    # a chunked prefill: the first step ends inside the second attention page and sends
    # page 0 only; the step that reaches the last token sends the rest and the GDN states
    first, last = [list(t) for t in w.tasks[:1]], [list(t) for t in w.tasks[:1]]
    first[0][:3] = [0, 1500, False]
    last[0][:3] = [1500, 4096 - 1500, True]
    w.tasks = first
    assert len(_oracle_lists(w)[0]) == 1
    _check_pack_unpack(w, seed=3)
    w.tasks = last
    assert int(_oracle_lists(w)[0][:, 2].sum()) == 6 * (2 << 20)
    _check_pack_unpack(w, seed=4)


def test_chunked_prefill_steps_and_ragged_tail():
    # two chunked-prefill steps of one request + a second request, ragged last block
    w = workloads.llama8b_single(n_layers=2, pool=64, tokens=100)
    src, dst = w.tasks[0][3], w.tasks[0][4]
    w.tasks = [[0, 37, False, src, dst], [37, 63, True, src, dst]]
    _check_pack_unpack(w)


def _transposing(w_t, seed=3, plan=None, lists=None):
    heads, ntpb, row = w_t.xform
    if plan is None:
        plan, lists = pipeline.build_plan(w_t, 0)
    runs = lists.tensor(0)
    B = 2 * heads * ntpb * row
    ids = np.concatenate([np.arange(r[0] // B, (r[0] + r[2]) // B) for r in runs]).astype(np.uint32)
    dst_ids = np.concatenate([np.arange(r[1] // B, (r[1] + r[2]) // B) for r in runs]).astype(np.uint32)
    src_layers = _make_caches(w_t, "src", seed)
    dst_layers = _make_caches(w_t, "dst", seed + 1, fill=False)
    sc = kvt_amd.Cache(0, src_layers, w_t.capacities("src"))
    dc = kvt_amd.Cache(0, dst_layers, w_t.capacities("dst"))
    stride = plan.layer_bytes
    packed = torch.zeros(w_t.n_layers * stride, dtype=torch.uint8, device="cuda")
    plan.pack(sc, 0, w_t.n_layers, packed, stride)
    plan.unpack(dc, 0, w_t.n_layers, packed, stride)
    torch.cuda.synchronize()
    lib = checkers.oracle()
    ph = _host(packed)
    for l in range(w_t.n_layers):
        hnd = _host(src_layers[l][0])
        blob = np.zeros(len(ids) * B, dtype=np.uint8)
        lib.kvto_pack_hnd_to_nhd(hnd.ctypes.data, ids.ctypes.data, len(ids), heads, ntpb, row,
                                 blob.ctypes.data)
        assert np.array_equal(ph[l * stride:l * stride + len(blob)], blob), l
        # same bytes as a plain pack of an NHD cache holding the same logical values
        nhd = np.ascontiguousarray(
            hnd.reshape(-1, 2, heads, ntpb, row).transpose(0, 1, 3, 2, 4)).reshape(-1)
        assert np.array_equal(blob, checkers.oracle_pack(nhd, runs))
        exp = np.full(w_t.capacities("dst")[0], 0xA5, dtype=np.uint8)
        lib.kvto_unpack_nhd_to_hnd(exp.ctypes.data, dst_ids.ctypes.data, len(ids), heads, ntpb,
                                   row, blob.ctypes.data)
        assert np.array_equal(_host(dst_layers[l][0]), exp), l
        # round trip: destination pages hold the source pages' bytes, still HND
        got = _host(dst_layers[l][0]).reshape(-1, B)
        assert np.array_equal(got[dst_ids], hnd.reshape(-1, B)[ids])


def test_config3_transposing_pack_hnd_to_nhd():
    _transposing(workloads.llama70b_flashinfer(n_layers=2, pool=128, n_req=3, tokens=500))


@pytest.mark.parametrize("heads,ntpb,row", [(1, 16, 256), (3, 5, 48), (8, 16, 16), (2, 64, 128)])
def test_transposing_pack_other_geometries(heads, ntpb, row):
    w = workloads.llama70b_flashinfer(n_layers=1, pool=40, n_req=2, tokens=3 * ntpb)
    T = 2 * heads * row
    for info in (w.src_info, w.dst_info):
        info["block_sizes"], info["token_sizes"], info["num_kv_heads"] = [T * ntpb], [T], heads
    rng = np.random.default_rng(5)
    w.tasks = [[0, 3 * ntpb, True, [[int(x) for x in rng.choice(40, 3, replace=False)]],
                [[int(x) for x in 3 * i + np.arange(3)]]] for i in range(2)]
    w.xform = (heads, ntpb, row)
    _transposing(w)


def test_arbitrary_ranges_including_misaligned():
    rng = np.random.default_rng(42)
    cap = 1 << 20
    runs, used = [], np.zeros(cap, dtype=bool)
    # destination ranges must not overlap (overlapping scatters race); largest first
    for ln in [70001, 257, 255, 17, 16, 15, 3, 2, 1] + list(rng.integers(1, 5000, size=200)):
        ln = int(ln)
        while True:
            d = int(rng.integers(0, cap - ln))
            if not used[d:d + ln].any():
                break
        used[d:d + ln] = True
        s = int(rng.integers(0, cap - ln))
        if rng.random() < 0.5:
            s &= ~15
        if rng.random() < 0.3:
            s = (s & ~15) | (d & 15)          # same misalignment on both sides
        runs.append((s, d, ln))
    runs = np.array(runs, dtype=np.uint64)
    lists = kvt_amd.BlockLists()
    lists.append(0, runs)
    plan = kvt_amd.Plan(0, lists, [cap], [cap], chunk_bytes=8192)
    src = _dev_bytes(cap, 9, "raw")
    dst = torch.full((cap,), 0x11, dtype=torch.uint8, device="cuda")
    sc, dc = kvt_amd.Cache(0, [[src]], [cap]), kvt_amd.Cache(0, [[dst]], [cap])
    packed = torch.zeros(plan.layer_bytes, dtype=torch.uint8, device="cuda")
    plan.pack(sc, 0, 1, packed, plan.layer_bytes)
    plan.unpack(dc, 0, 1, packed, plan.layer_bytes)
    torch.cuda.synchronize()
    blob = checkers.oracle_pack(_host(src), runs)
    assert np.array_equal(_host(packed)[:len(blob)], blob)
    exp = np.full(cap, 0x11, dtype=np.uint8)
    checkers.oracle_unpack(exp, runs, blob)
    assert np.array_equal(_host(dst), exp)


def test_plan_refuses_ranges_beyond_capacity_and_small_caches():
    lists = kvt_amd.BlockLists()
    lists.append(0, [(0, 0, 4096), (8192, 61440, 8192)])
    with pytest.raises(kvt_amd.KvtError) as e:
        kvt_amd.Plan(0, lists, [65536], [65536])
    assert e.value.code == 1
    plan = kvt_amd.Plan(0, lists, [65536], [131072])
    buf = torch.zeros(65536, dtype=torch.uint8, device="cuda")
    small = kvt_amd.Cache(0, [[buf]], [65536])
    packed = torch.zeros(plan.layer_bytes, dtype=torch.uint8, device="cuda")
    plan.pack(small, 0, 1, packed, plan.layer_bytes)          # source side fits
    with pytest.raises(kvt_amd.KvtError) as e:
        plan.unpack(small, 0, 1, packed, plan.layer_bytes)    # destination side does not
    assert e.value.code == 1
    with pytest.raises(kvt_amd.KvtError):
        plan.pack(small, 1, 1, packed, plan.layer_bytes)      # layer out of range
    torch.cuda.synchronize()


def test_cache_registration_checks_what_the_runtime_knows_about_the_memory():
    big = torch.zeros(64 << 20, dtype=torch.uint8, device="cuda")      # an allocation of its own
    kvt_amd.Cache(0, [[big]], [64 << 20]).close()
    kvt_amd.Cache(0, [[big[4096:]]], [(64 << 20) - 4096]).close()      # interior pointers are fine
    with pytest.raises(kvt_amd.KvtError) as e:
        kvt_amd.Cache(0, [[big]], [1 << 44])      # runs off any allocation (torch may have carved
        #                                             `big` out of a larger cached segment)
    assert e.value.code == 1 and "beyond the allocation" in str(e.value)
    host = np.zeros(1 << 16, dtype=np.uint8)
    with pytest.raises(kvt_amd.KvtError) as e:
        kvt_amd.Cache(0, [[host]], [1 << 16])                           # pageable host memory
    assert "cannot address" in str(e.value) or "can address" in str(e.value)
    pinned = torch.zeros(1 << 16, dtype=torch.uint8).pin_memory()
    kvt_amd.Cache(0, [[pinned]], [1 << 16]).close()                     # pinned host memory is legal
    # the packed buffer of a launch gets the same treatment
    lists = kvt_amd.BlockLists()
    lists.append(0, [(0, 0, 32 << 20)])
    plan = kvt_amd.Plan(0, lists, [64 << 20], [64 << 20])
    cache = kvt_amd.Cache(0, [[big], [big]], [64 << 20])
    packed = torch.zeros(48 << 20, dtype=torch.uint8, device="cuda")    # room for one layer only
    plan.pack(cache, 0, 1, packed, plan.layer_bytes)
    with pytest.raises(kvt_amd.KvtError) as e:
        plan.pack(cache, 0, 2, packed, 1 << 44)                         # layer 1 would land 16 TiB further
    assert e.value.code == 1 and "packed buffer" in str(e.value)
    with pytest.raises(kvt_amd.KvtError):
        plan.unpack(cache, 0, 1, np.zeros(32 << 20, dtype=np.uint8), plan.layer_bytes)
    torch.cuda.synchronize()


@pytest.mark.parametrize("n_ranges", [1, 63, 64, 65])
def test_short_plans_travel_in_the_kernel_arguments(n_ranges):
    """Up to 64 table entries are passed to the kernel by value, 65 take the resident table:
    the same bytes either way, also inside a stream capture taken right after creation (there
    is no table upload to wait for) and on two layers at once."""
    rng = np.random.default_rng(n_ranges)
    cap = 4 << 20
    slots = np.sort(rng.choice(cap // 32768, size=n_ranges, replace=False))
    lens = rng.integers(1, 32768, size=n_ranges)
    d_slots = rng.permutation(cap // 32768)[:n_ranges]
    ranges = np.stack([slots * 32768 + rng.integers(0, 3, size=n_ranges) * 16, d_slots * 32768,
                       lens], axis=1).astype(np.uint64)
    ranges[:, 2] = np.minimum(ranges[:, 2], 32768 - 48)
    lists = kvt_amd.BlockLists()
    lists.append(0, ranges)
    plan = kvt_amd.Plan(0, lists, [cap], [cap], chunk_bytes=32768)
    assert plan.num_chunks == n_ranges
    src = [[_dev_bytes(cap, 40 + l, "raw")] for l in range(2)]
    dst = [[torch.full((cap,), 0xA5, dtype=torch.uint8, device="cuda")] for l in range(2)]
    sc, dc = kvt_amd.Cache(0, src, [cap]), kvt_amd.Cache(0, dst, [cap])
    stride = plan.layer_bytes
    packed = torch.zeros(2 * stride, dtype=torch.uint8, device="cuda")
    s = checkers.side_stream()
    torch.cuda.synchronize()
    if n_ranges <= 64:
        graph = torch.cuda.CUDAGraph()
        torch.cuda.synchronize()          # what the default stream still holds comes first
        with torch.cuda.stream(s):
            with torch.cuda.graph(graph, stream=s):
                plan.pack(sc, 0, 2, packed, stride, s.cuda_stream)
                plan.unpack(dc, 0, 2, packed, stride, s.cuda_stream)
        graph.replay()
    else:
        plan.pack(sc, 0, 2, packed, stride, s.cuda_stream)
        plan.unpack(dc, 0, 2, packed, stride, s.cuda_stream)
    torch.cuda.synchronize()
    packed_h = _host(packed)
    for l in range(2):
        blob = checkers.oracle_pack(_host(src[l][0]), ranges)
        assert np.array_equal(packed_h[l * stride:l * stride + len(blob)], blob), l
        exp = np.full(cap, 0xA5, dtype=np.uint8)
        checkers.oracle_unpack(exp, ranges, blob)
        assert np.array_equal(_host(dst[l][0]), exp), l


def test_empty_plan_is_a_no_op():
    lists = kvt_amd.BlockLists()
    lists.append(0, np.zeros((0, 3), dtype=np.uint64))
    plan = kvt_amd.Plan(0, lists, [4096], [4096])
    assert plan.num_chunks == 0 and plan.layer_bytes == 0
    buf = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    plan.pack(kvt_amd.Cache(0, [[buf]], [4096]), 0, 1, buf, 0)
    torch.cuda.synchronize()


# ------------------------------------------------ reference-shaped entry points

def _soa(runs_contig_gpu_len):
    a = np.ascontiguousarray(runs_contig_gpu_len, dtype=np.int64)
    return [torch.from_numpy(np.ascontiguousarray(a[:, i])).cuda() for i in range(3)]


@pytest.mark.parametrize("n,maxlen", [(5, 200000), (300, 5000), (5000, 700)])
def test_launch_copy_direct_gather_and_scatter(n, maxlen):
    rng = np.random.default_rng(n)
    cap = 8 << 20
    lens = rng.integers(1, maxlen, size=n) // 16 * 16 + rng.choice([0, 16, 7], size=n)
    lens = np.maximum(lens, 1)
    gpu_off = np.sort(rng.choice(cap // 1024 - maxlen // 1024 - 2, size=n, replace=False)) * 1024
    lens = np.minimum(lens, np.diff(np.append(gpu_off, cap)))
    contig = np.concatenate([[0], np.cumsum(lens)[:-1]])
    total = int(lens.sum())
    src = _dev_bytes(cap, 77, "raw")
    out = torch.zeros(total, dtype=torch.uint8, device="cuda")
    so, do, ln = _soa(np.stack([gpu_off, contig, lens], axis=1))
    lib = kvt_amd.lib()
    rc = lib.kvt_launch_copy_d2h_direct(src.data_ptr(), out.data_ptr(), so.data_ptr(),
                                        do.data_ptr(), ln.data_ptr(), n, 0, 0, None)
    assert rc == 0, lib.kvt_last_error()
    torch.cuda.synchronize()
    runs = np.stack([gpu_off, gpu_off, lens], axis=1).astype(np.uint64)
    blob = checkers.oracle_pack(_host(src), runs)
    assert np.array_equal(_host(out), blob)
    dst = torch.full((cap,), 0x3C, dtype=torch.uint8, device="cuda")
    rc = lib.kvt_launch_copy_h2d_direct(out.data_ptr(), dst.data_ptr(), do.data_ptr(),
                                        so.data_ptr(), ln.data_ptr(), n, 64, 256, None)
    assert rc == 0, lib.kvt_last_error()
    torch.cuda.synchronize()
    exp = np.full(cap, 0x3C, dtype=np.uint8)
    checkers.oracle_unpack(exp, runs, blob)
    assert np.array_equal(_host(dst), exp)


@pytest.mark.parametrize("usage", [1.0, 0.25, 0.004], ids=["unlimited", "quarter", "eight-workgroups"])
def test_long_range_lists_go_through_the_persistent_range_kernels(usage):
    """A list of thousands of ranges is moved by persistent workgroups, a wavefront per range,
    8 KiB (converting: 4096 elements) per trip: ranges shorter, longer and much longer than a
    trip, empty ones, ranges that are not 16-byte aligned or not whole vectors long (copied on
    the spot), gather, scatter and the converting gather, against the oracle."""
    lib = kvt_amd.lib()
    o = checkers.oracle()
    rng = np.random.default_rng(4242)
    n, cap = 17000, 1088 << 20                            # unlimited: sixteen ranges per wavefront
    lens = rng.choice([0, 16, 48, 1000, 4096, 8192, 8208, 16384, 39936, 100000, 13, 4099], size=n,
                      p=[.03, .05, .05, .05, .2, .2, .1, .1, .1, .02, .05, .05]).astype(np.int64)
    slot = cap // n // 1024 * 1024                        # one slot per range: nothing overlaps
    gpu_off = np.arange(n, dtype=np.int64) * slot
    lens = np.minimum(lens, slot - 64)
    mis = rng.random(n) < 0.1
    gpu_off[mis] += rng.choice([1, 2, 4, 8], size=int(mis.sum()))
    order = rng.permutation(n)                            # the list is not sorted by address
    gpu_off, lens = gpu_off[order], lens[order]
    contig = np.concatenate([[0], np.cumsum(lens)[:-1]])
    contig16 = np.concatenate([[0], np.cumsum((lens + 15) // 16 * 16)[:-1]])   # aligned packed positions
    src = _dev_bytes(cap, 78, "raw")
    kvt_amd.set_copy_cu_usage(0, usage)
    try:
        for packed_off in (contig, contig16):
            total = int(packed_off[-1] + lens[-1])
            out = torch.zeros(total, dtype=torch.uint8, device="cuda")
            so, do, ln = _soa(np.stack([gpu_off, packed_off, lens], axis=1))
            assert lib.kvt_launch_copy_d2h_direct(src.data_ptr(), out.data_ptr(), so.data_ptr(),
                                                  do.data_ptr(), ln.data_ptr(), n, 0, 0, None) == 0
            torch.cuda.synchronize()
            src_h, out_h = _host(src), _host(out)
            exp = np.zeros(total, dtype=np.uint8)
            for g, p, l in zip(gpu_off, packed_off, lens):
                exp[p:p + l] = src_h[g:g + l]
            assert np.array_equal(out_h, exp)
            dst = torch.full((cap,), 0x3C, dtype=torch.uint8, device="cuda")
            assert lib.kvt_launch_copy_h2d_direct(out.data_ptr(), dst.data_ptr(), do.data_ptr(),
                                                  so.data_ptr(), ln.data_ptr(), n, 0, 0, None) == 0
            torch.cuda.synchronize()
            exp_d = np.full(cap, 0x3C, dtype=np.uint8)
            for g, p, l in zip(gpu_off, packed_off, lens):
                exp_d[g:g + l] = exp[p:p + l]
            assert np.array_equal(_host(dst), exp_d)
        # converting gather: lengths count elements, source offsets bytes of bf16
        elems = lens // 2
        e_off = np.concatenate([[0], np.cumsum((elems + 15) // 16 * 16 + 16)[:-1]])
        e_off[rng.random(n) < 0.05] += 4                  # some destinations not 16-byte aligned
        total_e = int(e_off[-1] + elems[-1])
        out8 = torch.zeros(total_e, dtype=torch.uint8, device="cuda")
        g_even = gpu_off // 2 * 2                          # bf16 elements start at even bytes
        so, do, ln = _soa(np.stack([g_even, e_off, elems], axis=1))
        assert lib.kvt_launch_copy_d2h_bf16_to_fp8(src.data_ptr(), out8.data_ptr(), so.data_ptr(),
                                                   do.data_ptr(), ln.data_ptr(), n, 0, 0, None) == 0
        torch.cuda.synchronize()
        table = np.array([o.kvto_bf16_to_fp8(int(b)) for b in range(65536)], dtype=np.uint8)
        src16 = _host(src).view(np.uint16)
        exp8 = np.zeros(total_e, dtype=np.uint8)
        for g, p, l in zip(g_even, e_off, elems):
            exp8[p:p + l] = table[src16[g // 2:g // 2 + l]]
        assert np.array_equal(_host(out8), exp8)
    finally:
        kvt_amd.set_copy_cu_usage(0, 1.0)


@pytest.mark.parametrize("n", [70000, 270000])
def test_very_long_lists_of_short_ranges_through_the_launchers(n):
    """From 65 536 ranges on a wavefront of the persistent range kernel moves two ranges side by
    side, from 262 144 on four: short ranges of every alignment, gather and scatter."""
    lib = kvt_amd.lib()
    rng = np.random.default_rng(n)
    slot = 1024
    cap = n * slot
    lens = rng.choice([16, 48, 256, 512, 1008, 13, 1000], size=n).astype(np.int64)
    gpu_off = (np.arange(n, dtype=np.int64) * slot)[rng.permutation(n)]
    gpu_off[rng.random(n) < 0.05] += 8
    contig = np.concatenate([[0], np.cumsum((lens + 15) // 16 * 16)[:-1]])
    total = int(contig[-1] + lens[-1])
    src = _dev_bytes(cap, 79, "raw")
    out = torch.zeros(total, dtype=torch.uint8, device="cuda")
    so, do, ln = _soa(np.stack([gpu_off, contig, lens], axis=1))
    assert lib.kvt_launch_copy_d2h_direct(src.data_ptr(), out.data_ptr(), so.data_ptr(),
                                          do.data_ptr(), ln.data_ptr(), n, 0, 0, None) == 0
    torch.cuda.synchronize()
    # expected: every range's bytes, by one fancy-indexed copy
    idx_src = np.concatenate([np.arange(g, g + l) for g, l in zip(gpu_off, lens)])
    idx_dst = np.concatenate([np.arange(p, p + l) for p, l in zip(contig, lens)])
    src_h = _host(src)
    exp = np.zeros(total, dtype=np.uint8)
    exp[idx_dst] = src_h[idx_src]
    assert np.array_equal(_host(out), exp)
    dst = torch.full((cap,), 0x3C, dtype=torch.uint8, device="cuda")
    assert lib.kvt_launch_copy_h2d_direct(out.data_ptr(), dst.data_ptr(), do.data_ptr(),
                                          so.data_ptr(), ln.data_ptr(), n, 0, 0, None) == 0
    torch.cuda.synchronize()
    exp_d = np.full(cap, 0x3C, dtype=np.uint8)
    exp_d[idx_src] = src_h[idx_src]
    assert np.array_equal(_host(dst), exp_d)


def test_reference_launcher_names_link_level_stand_in():
    """libkvt_blade_launchers.so exports the four extern "C" names that the reference's
    copy_kernels.cpp calls (copy_kernels.cpp:52-85, 101-108), with its argument order and a
    void return; called here the way that file calls them, persistent grid arguments included."""
    import ctypes as C
    import os
    lib = kvt_amd.lib()                                    # libkvt_hip.so first
    shim = C.CDLL(os.path.join(os.path.dirname(kvt_amd.LIB_PATH), "libkvt_blade_launchers.so"))
    vp, i64, ci = C.c_void_p, C.c_int64, C.c_int
    for name in ("launch_copy_d2h_direct_kernel", "launch_copy_h2d_direct_kernel",
                 "launch_copy_d2h_bf16_to_fp8_kernel"):
        fn = getattr(shim, name)
        fn.restype, fn.argtypes = None, [vp, vp, vp, vp, vp, i64, ci, ci, vp]
    shim.launch_copy_int64_array_h2d_kernel.restype = None
    shim.launch_copy_int64_array_h2d_kernel.argtypes = [vp, vp, i64, ci, ci, vp]

    n, cap = 700, 8 << 20
    rng = np.random.default_rng(12)
    lens = rng.integers(1, 300, size=n) * 16
    gpu_off = np.sort(rng.choice(cap // 8192, size=n, replace=False)) * 8192
    contig = np.concatenate([[0], np.cumsum(lens)[:-1]])
    total = int(lens.sum())
    src = _dev_bytes(cap, 5, "bf16")
    meta_h = torch.from_numpy(np.concatenate([gpu_off, contig, lens]).astype(np.int64)).pin_memory()
    meta_d = torch.zeros(3 * n, dtype=torch.int64, device="cuda")
    out = torch.zeros(total, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    s = checkers.side_stream()
    st = s.cuda_stream
    shim.launch_copy_int64_array_h2d_kernel(meta_h.data_ptr(), meta_d.data_ptr(), 3 * n, 2048, 512, st)
    so, do, ln = (meta_d.data_ptr() + 8 * n * k for k in range(3))
    shim.launch_copy_d2h_direct_kernel(src.data_ptr(), out.data_ptr(), so, do, ln, n, 2048, 512, st)
    s.synchronize()
    runs = np.stack([gpu_off, gpu_off, lens], axis=1).astype(np.uint64)
    blob = checkers.oracle_pack(_host(src), runs)
    assert np.array_equal(_host(out), blob)
    dst = torch.full((cap,), 0x3C, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    shim.launch_copy_h2d_direct_kernel(out.data_ptr(), dst.data_ptr(), do, so, ln, n, 2048, 512, st)
    s.synchronize()
    exp = np.full(cap, 0x3C, dtype=np.uint8)
    checkers.oracle_unpack(exp, runs, blob)
    assert np.array_equal(_host(dst), exp)
    # converting gather: lengths are element counts, destination offsets in fp8 bytes
    meta_h[n:2 * n] = torch.from_numpy((contig // 2).astype(np.int64))
    meta_h[2 * n:] = torch.from_numpy((lens // 2).astype(np.int64))
    out8 = torch.zeros(total // 2, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    shim.launch_copy_int64_array_h2d_kernel(meta_h.data_ptr(), meta_d.data_ptr(), 3 * n, 2048, 512, st)
    shim.launch_copy_d2h_bf16_to_fp8_kernel(src.data_ptr(), out8.data_ptr(), so, do, ln, n, 2048, 512, st)
    s.synchronize()
    want = torch.from_numpy(blob.copy()).view(torch.bfloat16).to(torch.float32).clamp(-448, 448) \
        .to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(_host(out8), want)
    # a refused call leaves a message, not a crash
    shim.launch_copy_d2h_direct_kernel(None, out.data_ptr(), so, do, ln, n, 1, 1, st)
    assert b"bad argument" in lib.kvt_last_error()


def test_start_up_profile_measures_both_copy_routes():
    """initialize_copy_method_profile (copy_kernels.cpp:495-591): loops of DMA copies against
    the copy kernel on pinned memory, once per process. What it finds must look like a PCIe
    part (tens of GB/s either way, microseconds of fixed cost), it decides the route unless the
    caller has set the thresholds, and either route gives the same bytes."""
    lib = kvt_amd.lib()
    assert lib.kvt_initialize_copy_method_profile(99) != 0
    assert lib.kvt_reset_copy_memcpy_thresholds() == 0
    d_fix, d_mib, k_fix, k_mib, ms = (C.c_double() for _ in range(5))
    single, measured = C.c_uint64(), C.c_int()
    for attempt in range(3):        # a disturbed measurement is discarded and may be repeated
        assert lib.kvt_initialize_copy_method_profile(0) == 0, lib.kvt_last_error()
        assert lib.kvt_get_copy_method_profile(0, None, None, None, None, None,
                                               C.byref(measured), None) == 0
        if measured.value:
            break
    for direction in (0, 1):
        assert lib.kvt_get_copy_method_profile(direction, C.byref(d_fix), C.byref(d_mib),
                                               C.byref(k_fix), C.byref(k_mib), C.byref(single),
                                               C.byref(measured), C.byref(ms)) == 0
        print("copy routes %s: DMA %.1f us + %.2f us/MiB, kernel %.1f us + %.2f us/MiB, own DMA "
              "copy from %d bytes (%.1f ms)" % ("H2D D2H".split()[direction], d_fix.value,
                                                d_mib.value, k_fix.value, k_mib.value,
                                                single.value, ms.value))
        assert measured.value == 1 and 0 < ms.value < 2000.0
        for per_mib in (d_mib.value, k_mib.value):          # 5 ... 87 GB/s across PCIe
            assert 12.0 < per_mib < 200.0, per_mib
        assert 0.0 <= d_fix.value < 500.0 and 0.0 <= k_fix.value < 500.0
        assert single.value >= 64 << 10                      # never worth it for small ranges
    # a second call measures nothing again; thresholds set by the caller win and can be undone
    assert lib.kvt_initialize_copy_method_profile(0) == 0
    assert lib.kvt_set_copy_memcpy_thresholds(3 << 20, 5) == 0
    assert lib.kvt_get_copy_method_profile(1, None, None, None, None, C.byref(single), None, None) == 0
    assert single.value == 3 << 20
    assert lib.kvt_reset_copy_memcpy_thresholds() == 0
    # the measured rule in charge: mixed lengths, bytes exact whichever way each range went
    _few_very_large_ranges(lib, expect_dma=False)


def test_copy_handle_data_hands_a_few_very_large_ranges_to_the_dma_engines():
    lib = kvt_amd.lib()
    assert lib.kvt_set_copy_memcpy_thresholds(8 << 20, 16) == 0
    try:
        _few_very_large_ranges(lib)
    finally:
        assert lib.kvt_reset_copy_memcpy_thresholds() == 0


def _few_very_large_ranges(lib, expect_dma=True):
    cap = 64 << 20
    lens = [(9 << 20) + 48, 8 << 20, (12 << 20) + 7]             # all >= 8 MiB, any remainder
    offs = [1 << 20, (12 << 20) + 16, (30 << 20) + 3]
    runs = np.array([[0, o, n] for o, n in zip(offs, lens)], dtype=np.uint64)
    total = int(sum(lens))
    layer = _dev_bytes(cap, 31, "raw")
    pinned = torch.zeros(total, dtype=torch.uint8).pin_memory()
    dev_meta = torch.zeros(3 * 8192, dtype=torch.int64, device="cuda")
    host_meta = torch.zeros(3 * 8192, dtype=torch.int64).pin_memory()
    s = checkers.side_stream()
    rc = lib.kvt_copy_handle_data_with_kernel(pinned.data_ptr(), layer.data_ptr(), runs.ctypes.data,
                                              len(runs), total, 1, 0, s.cuda_stream,
                                              dev_meta.data_ptr(), host_meta.data_ptr(), 0)
    assert rc == 0, lib.kvt_last_error()
    s.synchronize()
    gather = np.stack([runs[:, 1], runs[:, 1], runs[:, 2]], axis=1)
    blob = checkers.oracle_pack(_host(layer), gather)
    assert np.array_equal(pinned.numpy(), blob)
    dst = torch.full((cap,), 0x3C, dtype=torch.uint8, device="cuda")
    rc = lib.kvt_copy_handle_data_with_kernel(pinned.data_ptr(), dst.data_ptr(), runs.ctypes.data,
                                              len(runs), total, 0, 0, s.cuda_stream,
                                              dev_meta.data_ptr(), host_meta.data_ptr(), 0)
    assert rc == 0, lib.kvt_last_error()
    s.synchronize()
    exp = np.full(cap, 0x3C, dtype=np.uint8)
    checkers.oracle_unpack(exp, gather, blob)
    assert np.array_equal(_host(dst), exp)
    if expect_dma:
        assert (host_meta == 0).all()       # the kernel's metadata buffers were not needed


@pytest.mark.parametrize("n", [1, 2, 3, 511, 8192 * 3, 100001])
def test_launch_copy_int64_array_h2d(n):
    """launch_copy_int64_array_h2d_kernel of the reference (copy_kernels.cu:93-103): pinned
    int64 metadata read by a kernel, any count, also from an address that is only 8-byte
    aligned."""
    lib = kvt_amd.lib()
    rng = np.random.default_rng(n)
    host = torch.from_numpy(rng.integers(-2**62, 2**62, size=n + 1, dtype=np.int64)).pin_memory()
    dev = torch.full((n + 3,), -7, dtype=torch.int64, device="cuda")
    torch.cuda.synchronize()
    s = checkers.side_stream()
    for shift in (0, 1):
        rc = lib.kvt_launch_copy_int64_array_h2d(host.data_ptr() + 8 * shift, dev.data_ptr() + 8,
                                                 n, 0, 0, s.cuda_stream)
        assert rc == 0, lib.kvt_last_error()
        s.synchronize()
        got = dev.cpu()
        assert got[0] == -7 and (got[n + 1:] == -7).all()
        assert torch.equal(got[1:n + 1], host[shift:shift + n])
    assert lib.kvt_launch_copy_int64_array_h2d(host.data_ptr(), dev.data_ptr(), 0, 0, 0, None) == 0
    assert lib.kvt_launch_copy_int64_array_h2d(None, dev.data_ptr(), 4, 0, 0, None) != 0
    pageable = np.zeros(8, dtype=np.int64)                 # not device-visible: refused, no fault
    assert lib.kvt_launch_copy_int64_array_h2d(pageable.ctypes.data, dev.data_ptr(), 8, 0, 0, None) != 0


def test_memcpy_route_thresholds_decide_between_dma_and_kernel():
    """BLLM_KVTRANS_COPY_MEMCPY_{BLOCK_THRESHOLD_BYTES,MAX_BLOCKS} of the reference
    (copy_kernels.cpp:496-499, 610-617) as kvt_set_copy_memcpy_thresholds: the same three ranges
    of 1 MiB go through the kernel by default, to the DMA engines once the thresholds admit them,
    and through the kernel again when the route is switched off; the bytes never differ."""
    lib = kvt_amd.lib()
    cap = 16 << 20
    runs = np.array([[0, (1 << 20) + 32, 1 << 20], [0, 5 << 20, (1 << 20) + 5],
                     [0, (9 << 20) + 1, 1 << 20]], dtype=np.uint64)
    total = int(runs[:, 2].sum())
    layer = _dev_bytes(cap, 77, "raw")
    gather = np.stack([runs[:, 1], runs[:, 1], runs[:, 2]], axis=1)
    blob = checkers.oracle_pack(_host(layer), gather)
    dev_meta = torch.zeros(3 * 8192, dtype=torch.int64, device="cuda")
    s = checkers.side_stream()

    def gather_once():
        pinned = torch.zeros(total, dtype=torch.uint8).pin_memory()
        host_meta = torch.zeros(3 * 8192, dtype=torch.int64).pin_memory()
        rc = lib.kvt_copy_handle_data_with_kernel(pinned.data_ptr(), layer.data_ptr(),
                                                  runs.ctypes.data, len(runs), total, 1, 0,
                                                  s.cuda_stream, dev_meta.data_ptr(),
                                                  host_meta.data_ptr(), 0)
        assert rc == 0, lib.kvt_last_error()
        s.synchronize()
        assert np.array_equal(pinned.numpy(), blob)
        return bool((host_meta != 0).any())      # True: the kernel's metadata buffers were used

    try:
        assert lib.kvt_set_copy_memcpy_thresholds(8 << 20, 16) == 0   # the defaults, spelled out
        assert gather_once() is True
        assert lib.kvt_set_copy_memcpy_thresholds(1 << 20, 3) == 0
        assert gather_once() is False
        # one range too many for the whole-list rule; the lengths differ, so the per-range rule
        # of mixed lists still sends each of them to the DMA engines
        assert lib.kvt_set_copy_memcpy_thresholds(1 << 20, 2) == 0
        assert gather_once() is False
        assert lib.kvt_set_copy_memcpy_thresholds((1 << 20) + 1, 3) == 0   # two ranges too short
        assert gather_once() is True
        assert lib.kvt_set_copy_memcpy_thresholds(1, 0) == 0          # switched off
        assert gather_once() is True
    finally:
        assert lib.kvt_reset_copy_memcpy_thresholds() == 0


@pytest.mark.parametrize("max_block_num", [0, 2])
def test_mixed_lists_send_their_long_ranges_to_the_dma_engines(max_block_num):
    """enqueue_hybrid_copy of the reference (copy_kernels.cpp:675-722): in a list of mixed
    lengths the ranges at or above the threshold are copied one by one, the kernel gets the
    rest with their true positions in the contiguous buffer."""
    lib = kvt_amd.lib()
    cap = 16 << 20
    lens = [(1 << 20) + 32, 4096, 2 << 20, 65536 + 5, 4096, 1 << 20]
    offs = [0, 3 << 20, 4 << 20, 7 << 20, (8 << 20) + 3, 9 << 20]
    runs = np.array([[0, o, n] for o, n in zip(offs, lens)], dtype=np.uint64)
    total = int(sum(lens))
    layer = _dev_bytes(cap, 78, "raw")
    gather = np.stack([runs[:, 1], runs[:, 1], runs[:, 2]], axis=1)
    blob = checkers.oracle_pack(_host(layer), gather)
    dev_meta = torch.zeros(3 * 8192, dtype=torch.int64, device="cuda")
    host_meta = torch.zeros(3 * 8192, dtype=torch.int64).pin_memory()
    pinned = torch.zeros(total, dtype=torch.uint8).pin_memory()
    s = checkers.side_stream()
    try:
        assert lib.kvt_set_copy_memcpy_thresholds(1 << 20, 16) == 0
        rc = lib.kvt_copy_handle_data_with_kernel(pinned.data_ptr(), layer.data_ptr(),
                                                  runs.ctypes.data, len(runs), total, 1, 0,
                                                  s.cuda_stream, dev_meta.data_ptr(),
                                                  host_meta.data_ptr(), max_block_num)
        assert rc == 0, lib.kvt_last_error()
        s.synchronize()
        assert np.array_equal(pinned.numpy(), blob)
        # the kernel was given the three short ranges only (the last batch is still in the buffer)
        small = [(sum(lens[:i]), offs[i], lens[i]) for i in (1, 3, 4)]
        last = small if max_block_num == 0 else small[2:]
        m = len(last)
        got = host_meta[:3 * m].numpy().reshape(3, m).T.tolist()
        assert got == [list(t) for t in last]
        if max_block_num == 0:
            assert not host_meta[3 * m:64].any()
        else:                                     # the batch before it had two ranges
            assert not host_meta[6:64].any()
        dst = torch.full((cap,), 0x3C, dtype=torch.uint8, device="cuda")
        torch.cuda.synchronize()
        rc = lib.kvt_copy_handle_data_with_kernel(pinned.data_ptr(), dst.data_ptr(),
                                                  runs.ctypes.data, len(runs), total, 0, 0,
                                                  s.cuda_stream, dev_meta.data_ptr(),
                                                  host_meta.data_ptr(), max_block_num)
        assert rc == 0, lib.kvt_last_error()
        s.synchronize()
        exp = np.full(cap, 0x3C, dtype=np.uint8)
        checkers.oracle_unpack(exp, gather, blob)
        assert np.array_equal(_host(dst), exp)
    finally:
        assert lib.kvt_reset_copy_memcpy_thresholds() == 0


def test_copy_threads_get_their_own_metadata_buffers_and_streams():
    """get_kernel_copy_buffer / get_thread_local_{h2d,d2h}_stream of the reference's copy
    threads (copy_utils.cpp:9-154): per thread, created on first use, used for a real copy."""
    import threading
    lib = kvt_amd.lib()
    w = workloads.llama8b_single(n_layers=1, pool=64, tokens=300)
    runs = _oracle_lists(w)[0]
    cap = w.capacities("src")[0]
    layer = _dev_bytes(cap, 9)
    layer_h = _host(layer)
    total = int(runs[:, 2].sum())
    kb = np.stack([np.zeros(len(runs), dtype=np.uint64), runs[:, 0], runs[:, 2]], axis=1).copy()
    seen, errors = {}, []

    def work(i):
        try:
            dev, host, st, st2 = C.c_void_p(), C.c_void_p(), C.c_void_p(), C.c_void_p()
            assert lib.kvt_get_kernel_copy_buffer(0, 0, C.byref(dev), C.byref(host)) == 0
            d2, h2 = C.c_void_p(), C.c_void_p()
            assert lib.kvt_get_kernel_copy_buffer(0, 100, C.byref(d2), C.byref(h2)) == 0
            assert (d2.value, h2.value) == (dev.value, host.value)       # large enough already
            assert lib.kvt_get_thread_local_stream(0, 1, C.byref(st)) == 0
            assert lib.kvt_get_thread_local_stream(0, 1, C.byref(st2)) == 0 and st.value == st2.value
            assert lib.kvt_get_thread_local_stream(0, 0, C.byref(st2)) == 0 and st.value != st2.value
            pinned = torch.zeros(total, dtype=torch.uint8).pin_memory()
            rc = lib.kvt_copy_handle_data_with_kernel(pinned.data_ptr(), layer.data_ptr(),
                                                      kb.ctypes.data, len(kb), total, 1, 0, st,
                                                      dev, host, 0)
            assert rc == 0, lib.kvt_last_error()
            assert lib.kvt_stream_synchronize(st) == 0
            assert np.array_equal(pinned.numpy(), checkers.oracle_pack(layer_h, runs))
            seen[i] = (dev.value, host.value, st.value)
        except Exception as e:
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(3)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    assert len(seen) == 3
    bad = C.c_void_p()
    assert lib.kvt_get_thread_local_stream(0, 7, C.byref(bad)) != 0


def test_thread_stream_survives_a_larger_buffer_request():
    """A stream handed out stays valid when the same thread then asks for larger metadata
    buffers (only the buffers are replaced), and the copy through the new buffers on the old
    stream is exact."""
    lib = kvt_amd.lib()
    w = workloads.llama8b_single(n_layers=1, pool=64, tokens=300)
    runs = _oracle_lists(w)[0]
    cap = w.capacities("src")[0]
    layer = _dev_bytes(cap, 21)
    total = int(runs[:, 2].sum())
    kb = np.stack([np.zeros(len(runs), dtype=np.uint64), runs[:, 0], runs[:, 2]], axis=1).copy()
    st, st_after = C.c_void_p(), C.c_void_p()
    dev, host, dev2, host2 = C.c_void_p(), C.c_void_p(), C.c_void_p(), C.c_void_p()
    assert lib.kvt_get_thread_local_stream(0, 1, C.byref(st)) == 0
    assert lib.kvt_get_kernel_copy_buffer(0, 0, C.byref(dev), C.byref(host)) == 0
    assert lib.kvt_get_kernel_copy_buffer(0, 20000, C.byref(dev2), C.byref(host2)) == 0
    assert lib.kvt_get_thread_local_stream(0, 1, C.byref(st_after)) == 0
    assert st_after.value == st.value
    pinned = torch.zeros(total, dtype=torch.uint8).pin_memory()
    rc = lib.kvt_copy_handle_data_with_kernel(pinned.data_ptr(), layer.data_ptr(), kb.ctypes.data,
                                              len(kb), total, 1, 0, st, dev2, host2, 20000)
    assert rc == 0, lib.kvt_last_error()
    assert lib.kvt_stream_synchronize(st) == 0
    assert np.array_equal(pinned.numpy(), checkers.oracle_pack(_host(layer), runs))


def test_copy_handle_data_refuses_offsets_that_wrap():
    """offset + length beyond 64 bits is an error, not a small extent that passes the checks."""
    lib = kvt_amd.lib()
    layer = _dev_bytes(1 << 20, 3)
    pinned = torch.zeros(8192, dtype=torch.uint8).pin_memory()
    meta_d = torch.zeros(3 * 8192, dtype=torch.int64, device="cuda")
    meta_h = torch.zeros(3 * 8192, dtype=torch.int64).pin_memory()
    kb = np.array([[0, 0, 4096], [0, 2**64 - 2048, 4096]], dtype=np.uint64)
    rc = lib.kvt_copy_handle_data_with_kernel(pinned.data_ptr(), layer.data_ptr(), kb.ctypes.data,
                                              2, 8192, 1, 0, None, meta_d.data_ptr(),
                                              meta_h.data_ptr(), 0)
    assert rc == 1, lib.kvt_last_error()
    rc = lib.kvt_copy_handle_data_kernel_direct(pinned.data_ptr(), layer.data_ptr(), kb.ctypes.data,
                                                2, 8192, 1, 0, None, meta_d.data_ptr(),
                                                meta_d[8192:].data_ptr(), meta_d[16384:].data_ptr(),
                                                meta_h.data_ptr(), 0)
    assert rc == 1, lib.kvt_last_error()
    torch.cuda.synchronize()


@pytest.mark.parametrize("max_block_num", [0, 7])
def test_copy_handle_data_with_kernel_pinned_host_buffer(max_block_num):
    w = workloads.llama8b_single(n_layers=1, pool=64, tokens=300)
    runs = _oracle_lists(w)[0]
    cap = w.capacities("src")[0]
    layer = _dev_bytes(cap, 5)
    total = int(runs[:, 2].sum())
    pinned = torch.zeros(total, dtype=torch.uint8).pin_memory()
    n = len(runs)
    meta_n = 3 * max(n, 8192)
    dev_meta = torch.zeros(meta_n, dtype=torch.int64, device="cuda")
    host_meta = torch.zeros(meta_n, dtype=torch.int64).pin_memory()
    # sender convention: kernel blocks carry the GPU offset in dst_offset (tcp_channel.cpp:538-542)
    kb = np.stack([np.zeros(n, dtype=np.uint64), runs[:, 0], runs[:, 2]], axis=1).copy()
    lib = kvt_amd.lib()
    st = checkers.side_stream()
    rc = lib.kvt_copy_handle_data_with_kernel(pinned.data_ptr(), layer.data_ptr(), kb.ctypes.data,
                                              n, total, 1, 0, st.cuda_stream, dev_meta.data_ptr(),
                                              host_meta.data_ptr(), max_block_num)
    assert rc == 0, lib.kvt_last_error()
    st.synchronize()
    blob = checkers.oracle_pack(_host(layer), runs)
    assert np.array_equal(pinned.numpy(), blob)
    # receiver: scatter from the pinned buffer by dst_offset
    dst = torch.full((cap,), 0x77, dtype=torch.uint8, device="cuda")
    rb = np.ascontiguousarray(runs)
    rc = lib.kvt_copy_handle_data_with_kernel(pinned.data_ptr(), dst.data_ptr(), rb.ctypes.data, n,
                                              total, 0, 0, st.cuda_stream, dev_meta.data_ptr(),
                                              host_meta.data_ptr(), max_block_num)
    assert rc == 0, lib.kvt_last_error()
    st.synchronize()
    exp = np.full(cap, 0x77, dtype=np.uint8)
    checkers.oracle_unpack(exp, runs, blob)
    assert np.array_equal(_host(dst), exp)
    # wrong total is refused before anything is launched
    assert lib.kvt_copy_handle_data_with_kernel(pinned.data_ptr(), dst.data_ptr(), rb.ctypes.data,
                                                n, total + 1, 0, 0, None, dev_meta.data_ptr(),
                                                host_meta.data_ptr(), 0) == 3


def test_bf16_to_fp8_all_bit_patterns_and_converting_gather():
    lib = kvt_amd.lib()
    o = checkers.oracle()
    bits = np.arange(65536, dtype=np.uint16)
    src = torch.from_numpy(bits.view(np.int16).copy()).cuda()
    out = torch.zeros(65536, dtype=torch.uint8, device="cuda")
    so = torch.tensor([0, 2 * 40000], dtype=torch.int64, device="cuda")
    do = torch.tensor([0, 40000], dtype=torch.int64, device="cuda")
    ln = torch.tensor([40000, 25536], dtype=torch.int64, device="cuda")
    assert lib.kvt_launch_copy_d2h_bf16_to_fp8(src.data_ptr(), out.data_ptr(), so.data_ptr(),
                                               do.data_ptr(), ln.data_ptr(), 2, 0, 0, None) == 0
    torch.cuda.synchronize()
    exp = np.array([o.kvto_bf16_to_fp8(int(b)) for b in bits], dtype=np.uint8)
    assert np.array_equal(_host(out), exp)
    # unaligned element offsets take the scalar path
    so2 = torch.tensor([2 * 3], dtype=torch.int64, device="cuda")
    do2 = torch.tensor([5], dtype=torch.int64, device="cuda")
    ln2 = torch.tensor([1001], dtype=torch.int64, device="cuda")
    out2 = torch.zeros(2000, dtype=torch.uint8, device="cuda")
    assert lib.kvt_launch_copy_d2h_bf16_to_fp8(src.data_ptr(), out2.data_ptr(), so2.data_ptr(),
                                               do2.data_ptr(), ln2.data_ptr(), 1, 0, 0, None) == 0
    torch.cuda.synchronize()
    assert np.array_equal(_host(out2)[5:1006], exp[3:1004])
    # the "handle data" form: lengths are bf16 bytes, the pinned side gets half
    w = workloads.llama8b_single(n_layers=1, pool=32, tokens=200)
    runs = _oracle_lists(w)[0]
    layer = _dev_bytes(w.capacities("src")[0], 8)
    total = int(runs[:, 2].sum())
    pinned = torch.zeros(total // 2, dtype=torch.uint8).pin_memory()
    n = len(runs)
    dev_meta = torch.zeros(3 * 8192, dtype=torch.int64, device="cuda")
    host_meta = torch.zeros(3 * 8192, dtype=torch.int64).pin_memory()
    kb = np.stack([np.zeros(n, dtype=np.uint64), runs[:, 0], runs[:, 2]], axis=1).copy()
    assert lib.kvt_copy_d2h_bf16_to_fp8(pinned.data_ptr(), layer.data_ptr(), kb.ctypes.data, n,
                                        total, 0, None, dev_meta.data_ptr(), host_meta.data_ptr(),
                                        0) == 0
    torch.cuda.synchronize()
    fp8_runs = np.stack([runs[:, 0], runs[:, 1], runs[:, 2] // 2], axis=1).astype(np.uint64).copy()
    exp = np.zeros(total // 2, dtype=np.uint8)
    layer_h = _host(layer)
    o.kvto_pack_bf16_to_fp8(layer_h.ctypes.data, fp8_runs.ctypes.data, n, exp.ctypes.data)
    assert np.array_equal(pinned.numpy(), exp)


# ------------------------------------------------------- gating and staging

def test_per_layer_session_on_side_stream():
    w = workloads.llama8b_batch(n_layers=6, src_pool=256, dst_pool=256, n_req=3, min_tok=200,
                                max_tok=900)
    plan, lists = pipeline.build_plan(w, 0)
    layers = [[torch.zeros(w.capacities("src")[0], dtype=torch.uint8, device="cuda")]
              for _ in range(w.n_layers)]
    cache = kvt_amd.Cache(0, layers, w.capacities("src"))
    stride = plan.layer_bytes
    packed = torch.zeros(w.n_layers * stride, dtype=torch.uint8, device="cuda")
    sess = kvt_amd.Session(plan, cache, packed, stride)
    compute = checkers.side_stream()
    fresh = [_dev_bytes(w.capacities("src")[0], 50 + l) for l in range(w.n_layers)]
    torch.cuda.synchronize()          # what the default stream still holds comes first
    with torch.cuda.stream(compute):
        for l in range(w.n_layers):
            layers[l][0].copy_(fresh[l])           # the "forward pass" writes layer l
            sess.save_layer(l, compute.cuda_stream)
    for l in range(w.n_layers):
        sess.wait_layer(l)                         # what the transport thread does per layer
        blob = checkers.oracle_pack(_host(fresh[l]), lists.tensor(0))
        got = packed[l * stride:l * stride + len(blob)].cpu().numpy()
        assert np.array_equal(got, blob), l
    sess.join(compute.cuda_stream)
    compute.synchronize()
    sess.close()


def test_per_layer_session_gated_by_the_callers_own_events():
    """The reference's arrangement (blade_kvt/kv_transfer_impl.py:287-291, 320-327): the
    engine owns one event per layer, created once, and re-records event[layer] in every
    step; the library only ever sees the handles."""
    w = workloads.llama8b_batch(n_layers=5, src_pool=256, dst_pool=256, n_req=3, min_tok=200,
                                max_tok=900)
    plan, lists = pipeline.build_plan(w, 0)
    cap = w.capacities("src")[0]
    layers = [[torch.zeros(cap, dtype=torch.uint8, device="cuda")] for _ in range(w.n_layers)]
    cache = kvt_amd.Cache(0, layers, w.capacities("src"))
    stride = plan.layer_bytes
    packed = torch.zeros(w.n_layers * stride, dtype=torch.uint8, device="cuda")
    events = [torch.cuda.Event() for _ in range(w.n_layers)]
    compute = checkers.side_stream()
    for step in range(2):                          # the same events serve every step
        sess = kvt_amd.Session(plan, cache, packed, stride)
        fresh = [_dev_bytes(cap, 70 + 10 * step + l) for l in range(w.n_layers)]
        torch.cuda.synchronize()          # what the default stream still holds comes first
        with torch.cuda.stream(compute):
            for l in range(w.n_layers):
                layers[l][0].copy_(fresh[l])
                events[l].record(compute)
                sess.save_layer_event(l, events[l].cuda_event if l % 2 else events[l])
        for l in range(w.n_layers):
            sess.wait_layer(l)
            blob = checkers.oracle_pack(_host(fresh[l]), lists.tensor(0))
            got = packed[l * stride:l * stride + len(blob)].cpu().numpy()
            assert np.array_equal(got, blob), (step, l)
        sess.join(compute.cuda_stream)
        compute.synchronize()
        sess.close()
    with pytest.raises(kvt_amd.KvtError):
        kvt_amd.Session(plan, cache, packed, stride).save_layer_event(0, None)


def test_session_inside_hip_graph_replays():
    w = workloads.llama8b_single(n_layers=4, pool=64, tokens=200)
    plan, lists = pipeline.build_plan(w, 0)
    cap = w.capacities("src")[0]
    layers = [[torch.zeros(cap, dtype=torch.uint8, device="cuda")] for _ in range(w.n_layers)]
    staging = [torch.zeros(cap, dtype=torch.uint8, device="cuda") for _ in range(w.n_layers)]
    cache = kvt_amd.Cache(0, layers, [cap])
    stride = plan.layer_bytes
    packed = torch.zeros(w.n_layers * stride, dtype=torch.uint8, device="cuda")
    sess = kvt_amd.Session(plan, cache, packed, stride)
    graph = torch.cuda.CUDAGraph()
    s = checkers.side_stream()
    torch.cuda.synchronize()          # what the default stream still holds comes first
    with torch.cuda.stream(s):
        with torch.cuda.graph(graph, stream=s):
            for l in range(w.n_layers):
                layers[l][0].copy_(staging[l])
                sess.save_layer(l, s.cuda_stream)
            sess.join(s.cuda_stream)
    for rep in range(3):
        contents = [_dev_bytes(cap, 900 + 10 * rep + l) for l in range(w.n_layers)]
        for l in range(w.n_layers):
            staging[l].copy_(contents[l])
        packed.fill_(0)                                # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for l in range(w.n_layers):
            blob = checkers.oracle_pack(_host(contents[l]), lists.tensor(0))
            got = packed[l * stride:l * stride + len(blob)].cpu().numpy()
            assert np.array_equal(got, blob), (rep, l)
    sess.close()


def test_stager_save_load_round_trip_overlapped_with_packing():
    w = workloads.llama70b_flashinfer(n_layers=4, pool=64, n_req=2, tokens=300)
    plan, lists = pipeline.build_plan(w, 0)
    src_layers = _make_caches(w, "src", 21)
    dst_layers = _make_caches(w, "dst", 22, fill=False)
    sc = kvt_amd.Cache(0, src_layers, w.capacities("src"))
    dc = kvt_amd.Cache(0, dst_layers, w.capacities("dst"))
    nbytes = plan.layer_bytes
    stager = kvt_amd.Stager(0, nbytes, 2)
    dev_buf = [torch.zeros(nbytes, dtype=torch.uint8, device="cuda") for _ in range(2)]
    pack_stream = checkers.side_stream()
    store = []                                    # the "KV store": host copies per layer
    for l in range(w.n_layers):
        slot = l % 2
        if l >= 2:
            stager.wait(slot)                     # slot's previous D2H done -> consume it
            store.append(stager.slot_array(slot, nbytes).copy())
        plan.pack(sc, l, 1, dev_buf[slot], nbytes, pack_stream.cuda_stream)
        stager.save(slot, dev_buf[slot], nbytes, pack_stream.cuda_stream)
    for l in range(w.n_layers - 2, w.n_layers):
        stager.wait(l % 2)
        store.append(stager.slot_array(l % 2, nbytes).copy())
    o_runs = _oracle_lists(w)[0]
    assert np.array_equal(o_runs, lists.tensor(0))
    # what was stored is the NHD-ordered packed layer
    heads, ntpb, row = w.xform
    B = 2 * heads * ntpb * row
    ids = np.concatenate([np.arange(r[0] // B, (r[0] + r[2]) // B) for r in o_runs]).astype(np.uint32)
    lib = checkers.oracle()
    for l in range(w.n_layers):
        blob = np.zeros(len(ids) * B, dtype=np.uint8)
        src_h = _host(src_layers[l][0])
        lib.kvto_pack_hnd_to_nhd(src_h.ctypes.data, ids.ctypes.data, len(ids), heads, ntpb, row,
                                 blob.ctypes.data)
        assert np.array_equal(store[l][:len(blob)], blob), l
    # load path: host -> slot -> device -> unpack
    un_stream = checkers.side_stream()
    for l in range(w.n_layers):
        slot = l % 2
        stager.wait(slot)
        un_stream.synchronize()                   # device buffer of this slot is free again
        stager.slot_array(slot, nbytes)[:] = store[l]
        stager.load(slot, dev_buf[slot], nbytes, un_stream.cuda_stream)
        plan.unpack(dc, l, 1, dev_buf[slot], nbytes, un_stream.cuda_stream)
    un_stream.synchronize()
    dst_ids = np.concatenate([np.arange(r[1] // B, (r[1] + r[2]) // B) for r in o_runs]).astype(np.int64)
    ids = ids.astype(np.int64)
    for l in range(w.n_layers):
        got = _host(dst_layers[l][0]).reshape(-1, B)
        assert np.array_equal(got[dst_ids], _host(src_layers[l][0]).reshape(-1, B)[ids])
    stager.close()


def test_stager_loads_with_a_consumer_stream_per_slot():
    """Two device buffers, each with its own consumer stream and no host synchronisation with the
    kernels: a load into a buffer waits for the unpack that last read it, and only for that."""
    w = workloads.llama70b_flashinfer(n_layers=8, pool=96, n_req=3, tokens=400)
    plan, lists = pipeline.build_plan(w, 0)
    src_layers = _make_caches(w, "src", 31)
    dst_layers = _make_caches(w, "dst", 32, fill=False)
    sc = kvt_amd.Cache(0, src_layers, w.capacities("src"))
    dc = kvt_amd.Cache(0, dst_layers, w.capacities("dst"))
    nbytes = plan.layer_bytes
    packed = torch.zeros(w.n_layers * nbytes, dtype=torch.uint8, device="cuda")
    plan.pack(sc, 0, w.n_layers, packed, nbytes, 0)
    torch.cuda.synchronize()
    store = packed.cpu().numpy().reshape(w.n_layers, nbytes)
    stager = kvt_amd.Stager(0, nbytes, 2)
    dev_buf = [torch.zeros(nbytes, dtype=torch.uint8, device="cuda") for _ in range(2)]
    streams = [checkers.side_stream(), checkers.side_stream()]
    for l in range(w.n_layers):
        slot = l % 2
        if l >= 2:
            stager.wait(slot)                     # the slot's last transfer has left the host memory
        stager.slot_array(slot, nbytes)[:] = store[l]
        stager.load(slot, dev_buf[slot], nbytes, streams[slot].cuda_stream)
        plan.unpack(dc, l, 1, dev_buf[slot], nbytes, streams[slot].cuda_stream)
    streams[0].synchronize()
    streams[1].synchronize()
    o_runs = _oracle_lists(w)[0]
    heads, ntpb, row = w.xform
    B = 2 * heads * ntpb * row
    ids = np.concatenate([np.arange(r[0] // B, (r[0] + r[2]) // B) for r in o_runs]).astype(np.int64)
    dst_ids = np.concatenate([np.arange(r[1] // B, (r[1] + r[2]) // B) for r in o_runs]).astype(np.int64)
    for l in range(w.n_layers):
        got = _host(dst_layers[l][0]).reshape(-1, B)
        assert np.array_equal(got[dst_ids], _host(src_layers[l][0]).reshape(-1, B)[ids]), l
    stager.close()


def test_measure_pcie_reports_a_plausible_rate():
    lib = kvt_amd.lib()
    for direction in (0, 1):
        r = C.c_double()
        assert lib.kvt_measure_pcie(0, direction, 64 << 20, 3, C.byref(r)) == 0
        assert 1e9 < r.value < 2e11


def test_copy_linear():
    a = _dev_bytes((1 << 20) + 48, 1, "raw")
    b = torch.zeros_like(a)
    assert kvt_amd.lib().kvt_copy_linear(b.data_ptr(), a.data_ptr(), a.numel(), None) == 0
    torch.cuda.synchronize()
    assert torch.equal(a, b)


def test_plan_used_on_two_streams_then_destroyed_while_launches_are_queued():
    """The chunk table of a destroyed plan goes back to a pool; it must not be handed to the
    next plan while a kernel queued on ANY stream still reads it."""
    w = workloads.llama8b_batch(n_layers=24, src_pool=2048, dst_pool=3072, n_req=12, min_tok=500,
                                max_tok=2500)
    w2 = workloads.llama8b_batch(n_layers=24, src_pool=2048, dst_pool=3072, n_req=12, min_tok=500,
                                 max_tok=2500, seed=99)
    o_lists = _oracle_lists(w)
    src_layers = _make_caches(w, "src", 71)
    dst_layers = _make_caches(w, "dst", 72, fill=False)
    sc = kvt_amd.Cache(0, src_layers, w.capacities("src"))
    dc = kvt_amd.Cache(0, dst_layers, w.capacities("dst"))
    plan, _ = pipeline.build_plan(w, 0)
    stride = plan.layer_bytes
    packed = torch.zeros(w.n_layers * stride, dtype=torch.uint8, device="cuda")
    junk = torch.zeros(w.n_layers * stride * 2, dtype=torch.uint8, device="cuda")
    a, b = checkers.side_stream(), checkers.side_stream()
    plan.pack(sc, 0, w.n_layers, packed, stride, a.cuda_stream)
    done = torch.cuda.Event()
    done.record(a)
    b.wait_event(done)
    # keep stream a busy with a second, independent launch of the same plan, then use the
    # plan on stream b as well and drop it at once
    plan.pack(sc, 0, w.n_layers, junk, stride, a.cuda_stream)
    plan.unpack(dc, 0, w.n_layers, packed, stride, b.cuda_stream)
    plan.close()
    others = []
    for _ in range(4):       # same table size: the pool would hand the same storage out again
        p2, _ = pipeline.build_plan(w2, 0)
        p2.ready()
        others.append(p2)
    torch.cuda.synchronize()
    packed_h, junk_h = _host(packed), _host(junk)
    for l in range(w.n_layers):
        blob = checkers.oracle_pack(_host(src_layers[l][0]), o_lists[0])
        assert np.array_equal(packed_h[l * stride:l * stride + len(blob)], blob), l
        assert np.array_equal(junk_h[l * stride:l * stride + len(blob)], blob), l
        exp = np.full(w.capacities("dst")[0], 0xA5, dtype=np.uint8)
        checkers.oracle_unpack(exp, o_lists[0], blob)
        assert np.array_equal(_host(dst_layers[l][0]), exp), l
    for p2 in others:
        p2.close()


@pytest.mark.parametrize("explicit", [False, True])
def test_copy_handle_data_kernel_direct(explicit):
    """copy_handle_data_kernel_direct (copy_kernels.cpp:363-439): single batch, separate device
    arrays; the contiguous-side offset is the running sum, or blocks[i].src_offset when
    use_explicit_host_offsets is set."""
    rng = np.random.default_rng(12)
    cap, n = 1 << 20, 40
    lens = rng.integers(1, 6000, n).astype(np.uint64)
    gpu_off = (np.cumsum(lens + rng.integers(0, 5000, n).astype(np.uint64)) - lens).astype(np.uint64)
    assert int(gpu_off[-1] + lens[-1]) <= cap
    total = int(lens.sum())
    if explicit:      # contiguous side in shuffled order, with gaps
        order = rng.permutation(n)
        host_off = np.zeros(n, dtype=np.uint64)
        cur = 0
        for i in order:
            host_off[i] = cur
            cur += int(lens[i]) + int(rng.integers(0, 64))
        size = cur
    else:
        host_off = (np.cumsum(lens) - lens).astype(np.uint64)
        size = total
    blocks = np.ascontiguousarray(np.stack([host_off if explicit else np.zeros(n, np.uint64),
                                            gpu_off, lens], axis=1))
    layer = _dev_bytes(cap, 44, "u8")
    pinned = torch.zeros(size, dtype=torch.uint8).pin_memory()
    dev = [torch.zeros(n, dtype=torch.int64, device="cuda") for _ in range(3)]
    host_meta = torch.zeros(3 * n, dtype=torch.int64).pin_memory()
    lib = kvt_amd.lib()
    st = checkers.side_stream()

    def call(buf, gpu, direction, data_size=size):
        return lib.kvt_copy_handle_data_kernel_direct(
            buf.data_ptr(), gpu.data_ptr(), blocks.ctypes.data, n, data_size, direction, 0,
            st.cuda_stream, dev[0].data_ptr(), dev[1].data_ptr(), dev[2].data_ptr(),
            host_meta.data_ptr(), 1 if explicit else 0)

    assert call(pinned, layer, 1) == 0, lib.kvt_last_error()
    st.synchronize()
    layer_h, got = _host(layer), pinned.numpy()
    for i in range(n):
        a, b, m = int(host_off[i]), int(gpu_off[i]), int(lens[i])
        assert np.array_equal(got[a:a + m], layer_h[b:b + m]), i
    dst = torch.full((cap,), 0x33, dtype=torch.uint8, device="cuda")
    assert call(pinned, dst, 0) == 0, lib.kvt_last_error()
    st.synchronize()
    exp = np.full(cap, 0x33, dtype=np.uint8)
    for i in range(n):
        b, m = int(gpu_off[i]), int(lens[i])
        exp[b:b + m] = layer_h[b:b + m]
    assert np.array_equal(_host(dst), exp)
    # a range that leaves the contiguous buffer is refused before anything is launched
    assert call(pinned, dst, 0, data_size=int((host_off + lens).max()) - 1) != 0


@pytest.mark.parametrize("choice", [[16, 256, 1024, 4099, 48], [16, 256, 4096, 8192, 8208, 4099],
                                    [4096, 8192, 8208, 4099, 12000, 12272]], ids=["short", "medium", "long"])
@pytest.mark.parametrize("usage", [1.0, 0.25], ids=["unlimited", "quarter"])
def test_handle_data_between_two_device_buffers_with_a_long_list(usage, choice):
    """The contiguous side of copy_handle_data_kernel_direct and copy_handle_data_with_kernel
    may be device memory (a staging buffer registered for RDMA): a long list then takes the
    persistent range kernels like the device-array launchers. 20 000 ranges, some unaligned,
    gather and scatter, unlimited and under a limit."""
    rng = np.random.default_rng(13)
    n, slot = 20000, 12288
    cap = n * slot
    # (short: four ranges side by side per wavefront; medium: two; long: one)
    lens = rng.choice(choice, size=n).astype(np.uint64)
    gpu_off = (np.arange(n, dtype=np.uint64) * slot)[rng.permutation(n)]
    gpu_off[rng.random(n) < 0.05] += 4
    host_off = (np.cumsum(lens) - lens).astype(np.uint64)
    total = int(lens.sum())
    blocks = np.ascontiguousarray(np.stack([np.zeros(n, np.uint64), gpu_off, lens], axis=1))
    layer = _dev_bytes(cap, 45, "u8")
    staged = torch.zeros(total, dtype=torch.uint8, device="cuda")
    dev = [torch.zeros(n, dtype=torch.int64, device="cuda") for _ in range(3)]
    host_meta = torch.zeros(3 * n, dtype=torch.int64).pin_memory()
    dev_meta = torch.zeros(3 * 8192, dtype=torch.int64, device="cuda")
    lib = kvt_amd.lib()
    st = checkers.side_stream()
    layer_h = _host(layer)
    exp = np.zeros(total, dtype=np.uint8)
    for a, b, m in zip(host_off, gpu_off, lens):
        exp[int(a):int(a + m)] = layer_h[int(b):int(b + m)]
    exp_d = np.full(cap, 0x33, dtype=np.uint8)
    for b, m in zip(gpu_off, lens):
        exp_d[int(b):int(b + m)] = layer_h[int(b):int(b + m)]
    kvt_amd.set_copy_cu_usage(0, usage)
    try:
        for direct in (True, False):
            def call(gpu, direction):
                if direct:
                    return lib.kvt_copy_handle_data_kernel_direct(
                        staged.data_ptr(), gpu.data_ptr(), blocks.ctypes.data, n, total, direction, 0,
                        st.cuda_stream, dev[0].data_ptr(), dev[1].data_ptr(), dev[2].data_ptr(),
                        host_meta.data_ptr(), 0)
                return lib.kvt_copy_handle_data_with_kernel(
                    staged.data_ptr(), gpu.data_ptr(), blocks.ctypes.data, n, total, direction, 0,
                    st.cuda_stream, dev_meta.data_ptr(), host_meta.data_ptr(), 8192)
            staged.zero_()
            torch.cuda.synchronize()
            assert call(layer, 1) == 0, lib.kvt_last_error()
            st.synchronize()
            assert np.array_equal(_host(staged), exp), direct
            dst = torch.full((cap,), 0x33, dtype=torch.uint8, device="cuda")
            torch.cuda.synchronize()
            assert call(dst, 0) == 0, lib.kvt_last_error()
            st.synchronize()
            assert np.array_equal(_host(dst), exp_d), direct
    finally:
        kvt_amd.set_copy_cu_usage(0, 1.0)


_SKEWED = {
    # one range per wavefront
    "one": ([4096, 8192, 16384], [48 << 20, 48 << 20, (48 << 20) + 1000], (0, 4, 16)),
    # two side by side
    "two": ([4096, 4099, 2048], [(20 << 20) + 5, 300 << 10], (0, 1)),
    # four
    "four": ([256, 512, 1000, 13], [3 << 20, (1 << 20) + 7, 262145, 262144], (4, 0, 16, 1)),
    # more long ranges than the list of a launch holds (500): the rest stay with their owners
    "more than the list holds": ([4096, 8192], [(300 << 10) + 16 * k for k in range(600)],
                                 tuple(16 * (k % 3) for k in range(600))),
}


@pytest.mark.parametrize("shape,usage", [("one", 1.0), ("two", 1.0), ("four", 1.0),
                                         ("more than the list holds", 1.0), ("one", 0.25),
                                         ("more than the list holds", 0.25)])
def test_a_long_list_with_a_few_very_long_ranges(shape, usage, request):
    """Merged runs of many blocks among single blocks: 20 000 short ranges and a few of up to
    48 MiB, some of them not 16-byte aligned or not whole vectors long. A persistent
    wavefront's unit of work is a whole range; the ranges above 256 KiB are listed by the
    wavefronts that meet them and moved by a kernel behind, by all wavefronts together, in
    64 KiB segments. Through the host-list
    entry point (which sees the lengths), the device-array launchers (which do not) and the
    entry point that allocates nothing: the oracle's bytes, and the list takes at most three
    times what the same bytes take as even ranges (it took eight times that)."""
    short, longs, starts = _SKEWED[shape]
    request.addfinalizer(lambda: kvt_amd.set_copy_cu_usage(0, 1.0))
    kvt_amd.set_copy_cu_usage(0, usage)
    rng = np.random.default_rng(14)
    n, slot = 20000, 16384
    lens = rng.choice(short, size=n).astype(np.uint64)
    gpu_off = (np.arange(n, dtype=np.uint64) * slot)[rng.permutation(n)]
    gpu_off[rng.random(n) < 0.05] += 4
    where = rng.choice(n, size=len(longs), replace=False)  # the long ranges sit anywhere in the list
    at = n * slot
    for k, i in enumerate(where):
        lens[i] = longs[k]
        gpu_off[i] = at + starts[k]
        at += (longs[k] + 4096 + 255) // 256 * 256
    cap = int(at)
    host_off = (np.cumsum(lens) - lens).astype(np.uint64)
    total = int(lens.sum())
    blocks = np.ascontiguousarray(np.stack([np.zeros(n, np.uint64), gpu_off, lens], axis=1))
    layer = _dev_bytes(cap, 46, "raw")
    staged = torch.zeros(total, dtype=torch.uint8, device="cuda")
    dev = [torch.zeros(n, dtype=torch.int64, device="cuda") for _ in range(3)]
    host_meta = torch.zeros(3 * n, dtype=torch.int64).pin_memory()
    lib = kvt_amd.lib()
    st = checkers.side_stream()
    layer_h = _host(layer)
    idx_src = np.concatenate([np.arange(int(g), int(g + l)) for g, l in zip(gpu_off, lens)])
    exp = layer_h[idx_src]                                  # the packed side has no gaps
    exp_d = np.full(cap, 0x33, dtype=np.uint8)
    exp_d[idx_src] = exp

    def call(gpu, direction, blk=blocks, count=n, size=total):
        return lib.kvt_copy_handle_data_kernel_direct(
            staged.data_ptr(), gpu.data_ptr(), blk.ctypes.data, count, size, direction, 0,
            st.cuda_stream, dev[0].data_ptr(), dev[1].data_ptr(), dev[2].data_ptr(),
            host_meta.data_ptr(), 0)

    for _ in range(2):                                      # the second launch finds the block zeroed
        staged.zero_()
        torch.cuda.synchronize()
        assert call(layer, 1) == 0, lib.kvt_last_error()
        st.synchronize()
        assert np.array_equal(_host(staged), exp)
    dst = torch.full((cap,), 0x33, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    assert call(dst, 0) == 0, lib.kvt_last_error()
    st.synchronize()
    assert np.array_equal(_host(dst), exp_d)
    # the device-array launchers
    so, do, ln = _soa(np.stack([gpu_off, host_off, lens], axis=1).astype(np.int64))
    for _ in range(2):
        staged.zero_()
        assert lib.kvt_launch_copy_d2h_direct(layer.data_ptr(), staged.data_ptr(), so.data_ptr(),
                                              do.data_ptr(), ln.data_ptr(), n, 0, 0, None) == 0
        torch.cuda.synchronize()
        assert np.array_equal(_host(staged), exp)
    dst.fill_(0x33)
    assert lib.kvt_launch_copy_h2d_direct(staged.data_ptr(), dst.data_ptr(), do.data_ptr(),
                                          so.data_ptr(), ln.data_ptr(), n, 0, 0, None) == 0
    torch.cuda.synchronize()
    assert np.array_equal(_host(dst), exp_d)
    # the entry point that allocates nothing (8192 ranges at most): the first 7500 and the long ones
    keep = np.unique(np.concatenate([np.arange(7500), where]))
    sub = np.ascontiguousarray(blocks[keep])
    sub_total = int(sub[:, 2].sum())
    pinned_meta = torch.zeros(3 * len(keep), dtype=torch.int64).pin_memory()
    for _ in range(2):
        staged.zero_()
        torch.cuda.synchronize()
        assert lib.kvt_copy_handle_data_kernel_direct_static(
            staged.data_ptr(), layer.data_ptr(), sub.ctypes.data, len(keep), sub_total, 1, 0,
            st.cuda_stream, pinned_meta.data_ptr(), 0) == 0, lib.kvt_last_error()
        st.synchronize()
        idx_sub = np.concatenate([np.arange(int(g), int(g + l)) for g, l in zip(sub[:, 1], sub[:, 2])])
        assert np.array_equal(_host(staged)[:sub_total], layer_h[idx_sub])
    del dst

    # the same bytes as even ranges (every range 16 KiB) for the time
    m = total // 16384
    even = np.ascontiguousarray(np.stack([np.zeros(m, np.uint64), np.arange(m, dtype=np.uint64) * 16384,
                                          np.full(m, 16384, np.uint64)], axis=1))
    if m > n:
        dev = [torch.zeros(m, dtype=torch.int64, device="cuda") for _ in range(3)]
        host_meta = torch.zeros(3 * m, dtype=torch.int64).pin_memory()

    def timed(blk, count, size=total):
        best = 1e9
        for _ in range(4):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            with torch.cuda.stream(st):
                e0.record()
                assert call(layer, 1, blk, count, size) == 0, lib.kvt_last_error()
                e1.record()
            st.synchronize()
            best = min(best, e0.elapsed_time(e1))
        return best

    t_even, t_skew = timed(even, m, m * 16384), timed(blocks, n)
    print(f"skewed list {t_skew * 1e3:.0f} us, even list of the same bytes {t_even * 1e3:.0f} us")
    if len(longs) == 3:
        assert t_skew < 3 * t_even


def test_random_range_lists_sweep():
    """80 seeded batches of arbitrary ranges: 1-3 tensors, 1-3 layers, lengths from 1 byte to
    70 000, alignments 1 / 4 / 16 / 256, shuffled list order, every chunk size, packed buffer
    at a 16-, 4- or 1-byte aligned address."""
    for seed in range(80):
        rng = np.random.default_rng(10_000 + seed)
        n_t, n_layers = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        caps_s = [int(rng.integers(1 << 14, 1 << 20)) for _ in range(n_t)]
        caps_d = [int(rng.integers(1 << 14, 1 << 20)) for _ in range(n_t)]
        lists, all_runs = kvt_amd.BlockLists(), []
        for t in range(n_t):
            runs, d = [], 0
            align = int(rng.choice([1, 4, 16, 256]))
            while len(runs) <= 60:
                ln = int(rng.choice([1, 3, 16, 100, 4096, 5000, 40000, 70000]))
                ln = max(align, ln // align * align)
                gap = int(rng.integers(0, 4)) * align
                if d + gap + ln > caps_d[t] or ln > caps_s[t]:
                    break
                s = int(rng.integers(0, (caps_s[t] - ln) // align + 1)) * align
                runs.append((s, d + gap, ln))
                d += gap + ln
            runs = [runs[i] for i in rng.permutation(len(runs))] or [(0, 0, align)]
            lists.append(t, runs)
            all_runs.append(np.asarray(runs, np.uint64))
        chunk = int(rng.choice([0, 4096, 8192, 65536, 524288]))
        plan = kvt_amd.Plan(0, lists, caps_s, caps_d, chunk_bytes=chunk)
        src = [[_dev_bytes((c + 3) // 4 * 4, seed * 64 + l * 8 + t, "u8")[:c] for t, c in enumerate(caps_s)]
               for l in range(n_layers)]
        dst = [[torch.full((c,), 0xA5, device="cuda", dtype=torch.uint8) for c in caps_d]
               for _ in range(n_layers)]
        sc, dc = kvt_amd.Cache(0, src, caps_s), kvt_amd.Cache(0, dst, caps_d)
        pad = int(rng.choice([0, 0, 4, 1]))
        stride = plan.layer_bytes + 256
        packed = torch.zeros(n_layers * stride + 64, dtype=torch.uint8, device="cuda")
        plan.pack(sc, 0, n_layers, packed.data_ptr() + pad, stride)
        plan.unpack(dc, 0, n_layers, packed.data_ptr() + pad, stride)
        torch.cuda.synchronize()
        ph = _host(packed)[pad:]
        for l in range(n_layers):
            for t in range(n_t):
                blob = checkers.oracle_pack(_host(src[l][t]), all_runs[t])
                off = l * stride + plan.tensor_offset(t)
                assert np.array_equal(ph[off:off + len(blob)], blob), (seed, l, t, chunk, pad)
                exp = np.full(caps_d[t], 0xA5, dtype=np.uint8)
                checkers.oracle_unpack(exp, all_runs[t], blob)
                assert np.array_equal(_host(dst[l][t]), exp), (seed, l, t, chunk, pad)
        plan.close()


def test_transposing_pack_random_geometry_sweep():
    """30 seeded page geometries (heads 1-9, 1-70 tokens per page, rows of 16-1024 bytes, so
    also token rows longer than a slice) through the HND <-> NHD transform, each checked against
    the oracle's permutation, numpy's transpose and the round trip."""
    for seed in range(30):
        rng = np.random.default_rng(500 + seed)
        heads, ntpb = int(rng.integers(1, 10)), int(rng.integers(1, 71))
        row = 16 * int(rng.choice([1, 2, 3, 8, 16, 31, 64]))
        pool = int(rng.integers(6, 30))
        w = workloads.llama70b_flashinfer(n_layers=int(rng.integers(1, 3)), pool=pool, n_req=2,
                                          tokens=16)      # (tables are replaced below)
        T = 2 * heads * row
        for info in (w.src_info, w.dst_info):
            info["block_sizes"], info["token_sizes"], info["num_kv_heads"] = [T * ntpb], [T], heads
        src_ids = rng.permutation(pool)[:4]
        dst_ids = rng.permutation(pool)[:4]
        w.tasks = [[0, 2 * ntpb, True, [[int(x) for x in src_ids[2 * i:2 * i + 2]]],
                    [[int(x) for x in dst_ids[2 * i:2 * i + 2]]]] for i in range(2)]
        w.xform = (heads, ntpb, row)
        _transposing(w, seed=seed + 40)


def test_many_threads_build_launch_and_drop_plans_at_once():
    """The reference runs one sender thread per destination (kvtransfer/src/client.cpp:94-104).
    Here every thread parses its own batches, builds plans (the table pool and its upload
    stream are shared), packs from ONE registered cache on a stream of its own and drops the
    plan right after the launch. ctypes releases the GIL inside the library."""
    import threading
    n_threads, rounds = 6, 8
    base = workloads.llama8b_batch(n_layers=4, src_pool=1024, dst_pool=4096, n_req=4,
                                   min_tok=200, max_tok=1500)
    src_layers = _make_caches(base, "src", 81)
    sc = kvt_amd.Cache(0, src_layers, base.capacities("src"))
    src_h = [_host(src_layers[l][0]) for l in range(base.n_layers)]
    errors, checked = [], [0] * n_threads

    def work(i):
        try:
            stream = checkers.side_stream()
            for r in range(rounds):
                w = workloads.llama8b_batch(n_layers=4, src_pool=1024, dst_pool=4096, n_req=4,
                                            min_tok=200, max_tok=1500, seed=1000 + 17 * i + r)
                plan, lists = pipeline.build_plan(w, 0)
                stride = plan.layer_bytes
                packed = torch.zeros(w.n_layers * stride, dtype=torch.uint8, device="cuda")
                done = torch.cuda.Event()
                done.record()                       # the zero fill ran on the default stream
                stream.wait_event(done)
                plan.pack(sc, 0, w.n_layers, packed, stride, stream.cuda_stream)
                runs = lists.tensor(0)
                plan.close()                        # dropped while its launch may still be queued
                stream.synchronize()
                got = packed.cpu().numpy()
                for l in range(w.n_layers):
                    blob = checkers.oracle_pack(src_h[l], runs)
                    assert np.array_equal(got[l * stride:l * stride + len(blob)], blob), (i, r, l)
                checked[i] += 1
        except Exception as e:                      # an exception in a thread is otherwise lost
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(n_threads)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    assert checked == [rounds] * n_threads


@pytest.mark.parametrize("limit", [0, 1 << 40])
def test_either_load_flavour_moves_the_same_bytes(limit):
    """kvt_set_copy_cached_load_max: non-temporal loads always (0) or plain loads always (a huge
    limit) -- a plain table from the kernel arguments, a table in device memory, a transposing
    and a strided plan all give the oracle's bytes either way."""
    lib = kvt_amd.lib()
    assert lib.kvt_set_copy_cached_load_max(limit) == 0
    try:
        test_short_plans_travel_in_the_kernel_arguments(64)
        test_config2_shape_reduced_pool(0)
        test_config3_transposing_pack_hnd_to_nhd()
        test_config4_mla_and_indexer_two_tensors()
        test_arbitrary_ranges_including_misaligned()
    finally:
        assert lib.kvt_set_copy_cached_load_max(0) == 0


@pytest.mark.parametrize("loads", [0, 1 << 40])
def test_either_store_flavour_moves_the_same_bytes(loads):
    """kvt_set_copy_cached_store_max: plain stores for every launch between device buffers (a
    huge limit), with either load flavour -- the same plans give the oracle's bytes."""
    lib = kvt_amd.lib()
    assert lib.kvt_get_copy_cached_store_max() == 0
    assert lib.kvt_set_copy_cached_store_max(1 << 40) == 0 and lib.kvt_set_copy_cached_load_max(loads) == 0
    try:
        assert lib.kvt_get_copy_cached_store_max() == 1 << 40
        test_short_plans_travel_in_the_kernel_arguments(64)
        test_config2_shape_reduced_pool(0)
        test_config3_transposing_pack_hnd_to_nhd()
        test_config4_mla_and_indexer_two_tensors()
        test_arbitrary_ranges_including_misaligned()
    finally:
        assert lib.kvt_set_copy_cached_store_max(0) == 0 and lib.kvt_set_copy_cached_load_max(0) == 0
