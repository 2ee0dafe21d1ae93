"""Copy-plan tables checked without a GPU: a host-only plan (device = -1)
exposes the two chunk tables the kernels walk; a numpy emulation of the kernels'
addressing (same formulas as csrc/kvt_kernels.hip, with bounds asserted on
every access) must reproduce the CPU oracle's pack / unpack. Guards the table
builder -- above all that no entry can make a kernel touch memory outside the
registered tensors or the packed layer."""
import numpy as np
import pytest

import cases
import checkers
import kvt_amd
from kvt_amd import pipeline, workloads


_FP8_LUT = None


def _fp8_lut():
    global _FP8_LUT
    if _FP8_LUT is None:
        o = checkers.oracle()
        _FP8_LUT = np.array([o.kvto_bf16_to_fp8(b) for b in range(65536)], dtype=np.uint8)
    return _FP8_LUT


def emulate(table, chunk_bytes, shapes, caches, tensor_offset, packed, pack, convert=False):
    """convert (pack only): lengths count fp8 bytes = elements, the cache side holds bf16:
    a contiguous piece reads element e at byte 2e, a strided record 32 source bytes per
    16-byte output vector (convert_chunks_kernel)."""
    side = 0 if pack else 1
    scale = 2 if convert else 1
    assert pack or not convert
    touched = [np.zeros(len(c), dtype=bool) for c in caches]
    for c in table:
        n = int(c["len"])
        t = int(c["tensor"])
        assert 0 < n <= chunk_bytes
        pk0 = tensor_offset[t] + int(c["packed"])
        assert pk0 + n <= len(packed)
        if c["shape"] == 0:
            idx = int(c["cache"]) + np.arange(scale * n, dtype=np.int64)
            assert not convert or int(c["cache"]) % 2 == 0
        else:
            s = shapes[int(c["shape"]) - 1]
            vlen, inv, n_inner = int(s["vlen"]), int(s["inv_vlen"]), int(s["n_inner"])
            assert n % 16 == 0 and vlen > 0 and n_inner > 0
            assert int(c["cache"]) % 16 == 0 and pk0 % 16 == 0
            v = np.arange(n // 16, dtype=np.uint64)
            rec = v if vlen == 1 else (v * np.uint64(inv)) >> np.uint64(32)   # __umulhi
            assert np.array_equal(rec, v // np.uint64(vlen))                   # the reciprocal is exact
            w = np.arange(n // 4, dtype=np.uint64)                             # word-wise path
            assert np.array_equal((w * np.uint64(int(s["inv_wlen"]))) >> np.uint64(32),
                                  w // np.uint64(4 * vlen))
            inv_inner = int(s["inv_inner"])                                    # pipelined kernels
            if n_inner == 1:
                assert inv_inner == 0
            else:
                assert np.array_equal((rec * np.uint64(inv_inner)) >> np.uint64(32),
                                      rec // np.uint64(n_inner))
            col = v - rec * np.uint64(vlen)
            o, i = rec // np.uint64(n_inner), rec % np.uint64(n_inner)
            at = (o * np.uint64(int(s["outer"][side])) + i * np.uint64(int(s["inner"][side]))
                  + col * np.uint64(16 * scale)).astype(np.int64) + int(c["cache"])
            assert (at % 16 == 0).all()
            idx = (at[:, None] + np.arange(16 * scale, dtype=np.int64)[None, :]).reshape(-1)
        assert idx.min() >= 0 and idx.max() < len(caches[t]), "access outside the cache tensor"
        if convert:
            pairs = caches[t][idx].reshape(-1, 2).astype(np.uint32)
            packed[pk0:pk0 + n] = _fp8_lut()[pairs[:, 0] | (pairs[:, 1] << 8)]
        elif pack:
            packed[pk0:pk0 + n] = caches[t][idx]
        else:
            assert not touched[t][idx].any(), "two table entries write the same bytes"
            touched[t][idx] = True
            caches[t][idx] = packed[pk0:pk0 + n]


def _host_plan(lists_or_runs, s_cap, d_cap, chunk):
    return kvt_amd.Plan(-1, lists_or_runs, s_cap, d_cap, chunk_bytes=chunk)


def _check_tables(plan, o_lists, s_cap, d_cap, seed, unpack=True):
    pack_t, unpack_t, cb, shapes = plan.host_tables()
    n_t = len(o_lists)
    rng = np.random.default_rng(seed)
    src = [rng.integers(0, 256, c, dtype=np.uint8) for c in s_cap]
    offs = [plan.tensor_offset(t) for t in range(n_t)]
    packed = np.zeros(plan.layer_bytes, dtype=np.uint8)
    emulate(pack_t, cb, shapes, src, offs, packed, True)
    for t in range(n_t):
        blob = checkers.oracle_pack(src[t], o_lists[t])
        assert plan.tensor_bytes(t) == len(blob)
        assert np.array_equal(packed[offs[t]:offs[t] + len(blob)], blob), t
    # both tables hold the same entries up to order
    assert sorted(pack_t["packed"].tolist()) == sorted(unpack_t["packed"].tolist())
    for t in range(n_t):   # writes ascend: packed offset in the pack table, destination in the other
        sel = pack_t[pack_t["tensor"] == t]["packed"]
        assert (np.diff(sel.astype(np.int64)) > 0).all()
        sel = unpack_t[unpack_t["tensor"] == t]["cache"]
        assert (np.diff(sel.astype(np.int64)) >= 0).all()
    if unpack:
        dst = [np.full(c, 0xA5, dtype=np.uint8) for c in d_cap]
        emulate(unpack_t, cb, shapes, dst, offs, packed, False)
        for t in range(n_t):
            exp = np.full(d_cap[t], 0xA5, dtype=np.uint8)
            checkers.oracle_unpack(exp, o_lists[t], packed[offs[t]:offs[t] + plan.tensor_bytes(t)])
            assert np.array_equal(dst[t], exp), t


def _oracle_ranges(w):
    src, dst = w.worker_infos()
    rc, valid, tps, tpr, pid, kind = checkers.oracle_select(w.cache_shape, src, dst)
    rc, outs = checkers.oracle_parse(pid, src, dst, valid, tps, tpr, w.task_bufs())
    assert rc == 0
    if kind == 0:
        outs = [checkers.oracle_merge(o)[0] for o in outs]
    return outs


@pytest.mark.parametrize("chunk", [0, 4096, 16384, 524288])
@pytest.mark.parametrize("layout,p_tp,d_tp,rank", [("flash", 2, 1, 1), ("flash", 4, 1, 2),
                                                   ("ragged", 1, 2, 1), ("ragged", 4, 2, 3),
                                                   ("ragged", 1, 4, 0), ("hnd", 2, 1, 1)])
def test_run_plan_tables_for_tp_split_batches(layout, p_tp, d_tp, rank, chunk):
    w = workloads.tp_split(layout, p_tp, d_tp, rank, n_layers=1, src_pool=40, dst_pool=60,
                           n_req=4, min_tok=5, max_tok=150, total_heads=4, head_dim=32)
    src, dst = w.worker_infos()
    runs, _ = pipeline.parse_batch_runs(w.cache_shape, src, dst, w.task_bufs())
    plan = _host_plan(runs, w.capacities("src"), w.capacities("dst"), chunk)
    assert plan.num_strided_chunks > 0       # (the short head rows make "hnd" strided here too)
    _check_tables(plan, _oracle_ranges(w), w.capacities("src"), w.capacities("dst"), 7)


@pytest.mark.parametrize("parser", cases.ALL_PARSERS)
def test_run_plan_tables_for_random_cases_of_every_parser(parser):
    done = 0
    for seed in range(1200, 1320):
        case = cases.gen_case(parser, seed)
        pid, src, dst, valid, tps, tpr, tasks = cases.materialise(case)
        rc, outs = checkers.oracle_parse(pid, src, dst, valid, tps, tpr, tasks)
        if rc != 0 or not outs or any(len(o) == 0 for o in outs):
            continue
        parser_h = kvt_amd.Parser(pid, src, dst, valid, tps, tpr)
        runs = kvt_amd.RunLists()
        for t in tasks:
            assert parser_h.parse_runs(t.struct, runs) == 0
        n_t = runs.num_tensors()
        s_cap = [int(src.block_sizes[t]) * int(src.layer_num_blocks) for t in range(n_t)]
        d_cap = [int(dst.block_sizes[t]) * int(dst.layer_num_blocks) for t in range(n_t)]
        if max(s_cap + d_cap) > (64 << 20):
            continue
        plan = _host_plan(runs, s_cap, d_cap, [0, 4096, 32768][seed % 3])
        # the random cases may repeat destination blocks: gather only
        _check_tables(plan, outs, s_cap, d_cap, seed, unpack=False)
        # compressed plain lists give a second, independently built table
        lists = kvt_amd.BlockLists()
        for t, o in enumerate(outs):
            lists.append(t, o)
        plan2 = _host_plan(kvt_amd.RunLists.compress(lists), s_cap, d_cap, 0)
        _check_tables(plan2, outs, s_cap, d_cap, seed, unpack=False)
        done += 1
    assert done >= 10


@pytest.mark.parametrize("chunk", [0, 4096, 65536])
def test_plain_plan_tables_for_merged_batches(chunk):
    for w in (workloads.llama8b_batch(n_layers=1, src_pool=64, dst_pool=96, n_req=5, min_tok=10,
                                      max_tok=200),
              workloads.deepseek_mla(n_layers=1, pool=48, n_req=3, tokens=700)):
        src, dst = w.worker_infos()
        lists, _ = pipeline.parse_batch(w.cache_shape, src, dst, w.task_bufs())
        plan = _host_plan(lists, w.capacities("src"), w.capacities("dst"), chunk)
        assert plan.num_strided_chunks == 0
        _check_tables(plan, _oracle_ranges(w), w.capacities("src"), w.capacities("dst"), 9)


def test_hand_made_runs_three_levels_and_fallbacks():
    R = kvt_amd.RunLists()
    B = kvt_amd.BlockLists()
    rows = []
    # heads x tokens x (K,V): 3 x 5 x 2 records of 32 bytes
    for h in range(3):
        for tok in range(5):
            for kv in range(2):
                rows.append((64 + h * 2048 + tok * 64 + kv * 1024, 128 + h * 4096 + tok * 256 + kv * 128, 32))
    rows += [(8192, 16384, 8000)]                       # long plain range
    rows += [(20001 + 48 * i, 30000 + 100 * i, 20) for i in range(6)]   # misaligned: expanded
    B.append(0, rows)
    R = kvt_amd.RunLists.compress(B)
    assert R.tensor(0)[0]["n"].tolist() == [3, 5, 2]
    cap = [1 << 16]
    for chunk in (0, 4096, 8192):
        plan = _host_plan(R, cap, cap, chunk)
        assert plan.num_strided_chunks == 3             # one per head
        _check_tables(plan, [np.asarray(rows, np.uint64)], cap, cap, 3)


def test_run_plan_rejects_runs_beyond_capacity():
    B = kvt_amd.BlockLists()
    B.append(0, [(0 + 64 * i, 0 + 64 * i, 32) for i in range(8)])
    R = kvt_amd.RunLists.compress(B)
    assert len(R.tensor(0)) == 1
    kvt_amd.Plan(-1, R, [480], [480]).close()
    with pytest.raises(kvt_amd.KvtError):
        kvt_amd.Plan(-1, R, [479], [480])
    with pytest.raises(kvt_amd.KvtError):
        kvt_amd.Plan(-1, R, [480], [479])
    with pytest.raises(kvt_amd.KvtError):              # a host-only plan cannot be launched
        kvt_amd.lib().kvt_pack.restype
        p = kvt_amd.Plan(-1, R, [480], [480])
        kvt_amd.binding.check(kvt_amd.lib().kvt_pack(p.h, None, 0, 1, None, 0, None))


@pytest.mark.parametrize("seed", range(25))
def test_run_plan_tables_for_random_synthetic_runs(seed):
    """Runs that no parser would emit: odd lengths, zero strides on the source side,
    three full levels, lengths around the 4 KiB limit, many distinct shapes (more than the
    16 the kernel takes by value: the rest must fall back to plain chunks)."""
    cap = 1 << 22
    runs = cases.gen_synthetic_runs(seed, cap, kvt_amd.binding.RUN_DTYPE)
    R = kvt_amd.RunLists()
    R.append(0, runs)
    expect = R.expand().tensor(0)
    from test_runs import numpy_expand
    assert np.array_equal(expect, numpy_expand(runs))
    for chunk in (0, 4096, 65536):
        plan = _host_plan(R, [cap], [cap], chunk)
        _check_tables(plan, [expect], [cap], [cap], seed)


def test_run_lists_append_refuses_empty_runs():
    bad = np.zeros(1, dtype=kvt_amd.binding.RUN_DTYPE)
    bad["length"], bad["n"] = 16, [[1, 0, 1]]
    with pytest.raises(kvt_amd.KvtError):
        kvt_amd.RunLists().append(0, bad)


@pytest.mark.parametrize("chunk", [0, 4096, 65536])
@pytest.mark.parametrize("layout,p_tp,d_tp,rank", [("flash", 2, 1, 1), ("flash", 4, 1, 2),
                                                   ("ragged", 4, 1, 3)])
def test_converting_plan_tables_bf16_sender_fp8_receiver(layout, p_tp, d_tp, rank, chunk):
    w = workloads.tp_split(layout, p_tp, d_tp, rank, n_layers=1, src_pool=40, dst_pool=60,
                           n_req=4, min_tok=5, max_tok=150, total_heads=4, head_dim=32,
                           fp8_dst=True)
    src, dst = w.worker_infos()
    runs, _ = pipeline.parse_batch_runs(w.cache_shape, src, dst, w.task_bufs(), fp8=True)
    s_cap, d_cap = w.capacities("src"), w.capacities("dst")
    plan = kvt_amd.Plan(-1, runs, s_cap, d_cap, chunk_bytes=chunk, bf16_to_fp8=True)
    assert plan.num_strided_chunks > 0
    rc, valid, tps, tpr, pid, kind = checkers.oracle_select(w.cache_shape, src, dst)
    rc, outs = checkers.oracle_parse(pid, src, dst, valid, tps, tpr, w.task_bufs(), fp8=True)
    assert rc == 0 and np.array_equal(runs.expand().tensor(0), outs[0])
    ranges = np.ascontiguousarray(outs[0], dtype=np.uint64)
    pack_t, unpack_t, cb, shapes = plan.host_tables()
    rng = np.random.default_rng(11)
    cache = rng.integers(0, 256, s_cap[0], dtype=np.uint8)
    packed = np.zeros(plan.layer_bytes, dtype=np.uint8)
    emulate(pack_t, cb, shapes, [cache], [plan.tensor_offset(0)], packed, True, convert=True)
    blob = np.zeros(int(ranges[:, 2].sum()), dtype=np.uint8)
    checkers.oracle().kvto_pack_bf16_to_fp8(cache.ctypes.data, ranges.ctypes.data, len(ranges),
                                            blob.ctypes.data)
    assert plan.tensor_bytes(0) == len(blob) and np.array_equal(packed[:len(blob)], blob)
    dst_c = [np.full(d_cap[0], 0xA5, dtype=np.uint8)]
    emulate(unpack_t, cb, shapes, dst_c, [plan.tensor_offset(0)], packed, False)
    exp = np.full(d_cap[0], 0xA5, dtype=np.uint8)
    checkers.oracle_unpack(exp, ranges, blob)
    assert np.array_equal(dst_c[0], exp)


def test_converting_plan_checks_the_source_at_twice_the_length_and_on_element_bounds():
    cap_s, cap_d = 1 << 20, 1 << 19
    edge = kvt_amd.BlockLists()
    edge.append(0, [(cap_s - 64, 0, 64)])
    kvt_amd.Plan(-1, kvt_amd.RunLists.compress(edge), [cap_s], [cap_d]).close()
    with pytest.raises(kvt_amd.KvtError) as e:
        kvt_amd.Plan(-1, kvt_amd.RunLists.compress(edge), [cap_s], [cap_d], bf16_to_fp8=True)
    assert e.value.code == 1
    odd = kvt_amd.BlockLists()
    odd.append(0, [(3, 0, 64)])
    with pytest.raises(kvt_amd.KvtError) as e:
        kvt_amd.Plan(-1, kvt_amd.RunLists.compress(odd), [cap_s], [cap_d], bf16_to_fp8=True)
    assert e.value.code == 3
    # plain pieces: the k-th chunk of a long range starts 2 * k * chunk_bytes into the source
    long = kvt_amd.BlockLists()
    long.append(0, [(4096, 128, 100000)])
    plan = kvt_amd.Plan(-1, kvt_amd.RunLists.compress(long), [cap_s], [cap_d], chunk_bytes=32768,
                        bf16_to_fp8=True)
    pack_t, unpack_t, cb, _ = plan.host_tables()
    assert pack_t["cache"].tolist() == [4096 + 2 * 32768 * k for k in range(4)]
    assert unpack_t["cache"].tolist() == [128 + 32768 * k for k in range(4)]
