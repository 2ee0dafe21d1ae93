"""Product ParseBlock (kvt_parse_block of libkvt_hip.so, host code) against the
CPU oracle and the golden vectors of the compiled reference. CPU-only tests."""
import json
import os

import numpy as np
import pytest

import cases
import checkers
import kvt_amd
from kvt_amd.ctypes_defs import PARSER, TaskBuf, make_worker_info

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "parse_golden.json")
with open(GOLDEN) as f:
    _GOLDEN = json.load(f)


def product_parse(case, pad=True):
    """-> (rc, [per-tensor (n,3) arrays]) through the C ABI of the product library"""
    pid, src, dst, valid, tps, tpr, tasks = cases.materialise(case)
    parser = kvt_amd.Parser(pid, src, dst, valid, tps, tpr, fp8=case["fp8"], pad=pad)
    lists = kvt_amd.BlockLists()
    for t in tasks:
        rc = parser.parse(t.struct, lists)
        if rc != 0:
            return rc, []
    return 0, lists.all()


def _same(a_list, b_list, name):
    assert len(a_list) == len(b_list), name
    for t, (a, b) in enumerate(zip(a_list, b_list)):
        a = np.asarray(a, dtype=np.uint64).reshape(-1, 3)
        b = np.asarray(b, dtype=np.uint64).reshape(-1, 3)
        assert a.shape == b.shape, (name, t, a.shape, b.shape)
        assert np.array_equal(a, b), (name, t)


@pytest.mark.parametrize("case", _GOLDEN, ids=[c["name"] for c in _GOLDEN])
def test_product_matches_reference_golden(case):
    rc, outs = product_parse(case)
    assert rc == case["rc"]
    if rc == 0:
        _same(outs, case["expect"], case["name"])


@pytest.mark.parametrize("parser", cases.ALL_PARSERS)
def test_product_matches_oracle_on_random_cases(parser):
    emitted = 0
    for seed in range(200, 400):
        case = cases.gen_case(parser, seed)
        pid, src, dst, valid, tps, tpr, tasks = cases.materialise(case)
        rc_o, out_o = checkers.oracle_parse(pid, src, dst, valid, tps, tpr, tasks)
        rc_p, out_p = product_parse(case)
        assert rc_p == rc_o, case["name"]
        _same(out_p, out_o, case["name"])
        emitted += sum(len(o) for o in out_p)
    assert emitted > 0


@pytest.mark.parametrize("parser", ["RAGGED_PGTD", "RAGGED_PLTD", "FLASH_PGTD", "DPSK_PGTD",
                                    "DPSK_PLTD", "FLASH_PEQD"])
def test_product_matches_oracle_with_fp8_conversion(parser):
    for seed in range(500, 560):
        case = cases.gen_case(parser, seed)
        case["fp8"] = True
        pid, src, dst, valid, tps, tpr, tasks = cases.materialise(case)
        rc_o, out_o = checkers.oracle_parse(pid, src, dst, valid, tps, tpr, tasks, fp8=True)
        rc_p, out_p = product_parse(case)
        assert rc_p == rc_o, case["name"]
        if rc_o == 0:
            _same(out_p, out_o, case["name"])


@pytest.mark.parametrize("parser", ["HYBRID_PGTD", "HYBRID_PLTD", "HYBRID_FI_PGTD",
                                    "HYBRID_FI_PLTD"])
def test_product_matches_oracle_without_tail_padding(parser):
    # the reference cannot switch BLLM_KVTRANS_PAD_LAST_ATTN_BLOCK off (its env
    # reader maps "0" to the default), so this is pinned by the oracle alone
    for seed in range(600, 660):
        case = cases.gen_case(parser, seed)
        pid, src, dst, valid, tps, tpr, tasks = cases.materialise(case)
        rc_o, out_o = checkers.oracle_parse(pid, src, dst, valid, tps, tpr, tasks, pad=False)
        rc_p, out_p = product_parse(case, pad=False)
        assert rc_p == rc_o
        _same(out_p, out_o, case["name"])


@pytest.mark.parametrize("parser", ["RAGGED_PEQD", "FLASH_PEQD", "DPSK_PEQD", "FLASHINFER_PEQD",
                                    "HYBRID_PEQD", "RAGGED_PGTD", "FLASH_PGTD", "HYBRID_FI_PGTD"])
def test_out_of_pool_block_ids_are_rejected(parser):
    hits = 0
    for seed in range(40):
        case = cases.gen_case(parser, 1000 + seed)
        t = case["tasks"][0]
        g = len(t[4]) - 1
        while g >= 0 and not t[4][g]:
            g -= 1
        t[4][g][0] = case["dst"]["layer_num_blocks"] + 3
        pid, src, dst, valid, tps, tpr, tasks = cases.materialise(case)
        rc_o, _ = checkers.oracle_parse(pid, src, dst, valid, tps, tpr, tasks)
        rc_p, _ = product_parse(case)
        assert rc_p == rc_o, case["name"]
        hits += rc_p != 0
    assert hits > 0
    assert "range validation" in kvt_amd.lib().kvt_last_error().decode() or hits


def test_too_short_block_table_is_out_of_range():
    w = make_worker_info([65536], [4096], 64)
    parser = kvt_amd.Parser(PARSER["FLASH_PEQD"], w, w, 1, 1, 0)
    lists = kvt_amd.BlockLists()
    assert parser.parse(TaskBuf(0, 40, True, [[1, 2]], [[3, 4]]).struct, lists) == 1


def test_capacity_overflow_and_missing_tensor():
    big = make_worker_info([2**63], [2**20], 4)
    parser = kvt_amd.Parser(PARSER["RAGGED_PEQD"], big, big, 1, 1, 0)
    assert parser.parse(TaskBuf(0, 1, True, [[0]], [[0]]).struct, kvt_amd.BlockLists()) == 2
    src = make_worker_info([36864, 8192], [576, 128], 8)
    dst = make_worker_info([36864], [576], 8)
    parser = kvt_amd.Parser(PARSER["DPSK_PEQD"], src, dst, 1, 1, 0)
    assert parser.parse(TaskBuf(0, 1, True, [[0]], [[0]]).struct, kvt_amd.BlockLists()) == 1
    rc_o, _ = checkers.oracle_parse(PARSER["DPSK_PEQD"], src, dst, 1, 1, 0,
                                    [TaskBuf(0, 1, True, [[0]], [[0]])])
    assert rc_o == 1


@pytest.mark.parametrize("shape", [1, 2, 3, 4, 5, 6, 7, 8])
def test_select_parser_matches_oracle(shape):
    rng = np.random.default_rng(shape)
    for _ in range(200):
        p_tp = int(rng.choice([1, 2, 4, 8, 16]))
        d_tp = int(rng.choice([1, 2, 4, 8, 16]))
        heads = int(rng.choice([-1, 1, 2, 4, 8, 16, 32]))
        big, small = max(p_tp, d_tp), min(p_tp, d_tp)
        if heads > 0 and (big % heads and heads % big):
            continue
        rank = int(rng.integers(0, p_tp))
        same = bool(rng.random() < 0.5)
        src = make_worker_info([4096 * 16], [4096], 8, tp=p_tp, rank=rank, num_kv_heads=heads)
        dst = make_worker_info([4096 * 16] if same else [8192 * 16], [4096] if same else [8192], 8,
                               tp=d_tp, rank=0, num_kv_heads=heads)
        rc_o, *exp = checkers.oracle_select(shape, src, dst)
        try:
            got = kvt_amd.select_parser(shape, src, dst)
            assert rc_o == 0 and tuple(exp) == got
        except kvt_amd.KvtError as e:
            assert rc_o == e.code == 4


def test_select_parser_unknown_shape():
    w = make_worker_info([16384], [1024], 8)
    with pytest.raises(kvt_amd.KvtError) as e:
        kvt_amd.select_parser(42, w, w)
    assert e.value.code == 4 and "unsupported cache_shape" in str(e.value)


@pytest.mark.parametrize("p,d,heads,mask", [
    (4, 2, 8, 0b1111), (8, 4, 8, 0xFF), (8, 4, -1, 0xFF), (8, 2, 2, 0b00010001),
    (8, 2, 4, 0b01010101), (8, 4, 2, 0b01010101), (2, 8, 4, 0b11), (4, 2, 2, 0b0101),
])
def test_valid_ranks_known_answers(p, d, heads, mask):
    # numbers asserted by the reference: kvtransfer/tests/send_stub_test.cpp:2739-2802
    assert kvt_amd.compute_valid_ranks_pd(p, d, heads) == mask


@pytest.mark.parametrize("data,merged,stats", [
    ([], [], (2**64 - 1, 0, 0, 0)),
    ([(1, 1, 1)], [(1, 1, 1)], (1, 1, 1, 1)),
    ([(1, 1, 1), (3, 3, 2)], [(1, 1, 1), (3, 3, 2)], (1, 2, 3, 2)),
    ([(1, 1, 2), (3, 3, 1)], [(1, 1, 3)], (3, 3, 3, 1)),
    ([(1, 1, 2), (3, 3, 1), (4, 5, 2)], [(1, 1, 3), (4, 5, 2)], (2, 3, 5, 2)),
    ([(1, 1, 2), (1, 3, 1), (2, 4, 2)], [(1, 1, 2), (1, 3, 3)], (2, 3, 5, 2)),
])
def test_merge_known_answers(data, merged, stats):
    # kvtransfer/tests/send_stub_test.cpp:1212-1277
    got, st = kvt_amd.merge_interval(np.array(data, dtype=np.uint64).reshape(-1, 3))
    assert [tuple(r) for r in got.tolist()] == merged
    assert st == stats


def test_merge_matches_oracle_on_random_lists():
    rng = np.random.default_rng(11)
    for _ in range(200):
        n = int(rng.integers(0, 60))
        # build lists with plenty of adjacency: consecutive pieces, shuffled
        pieces, s, d = [], 0, 1000
        for _i in range(n):
            ln = int(rng.integers(1, 9))
            if rng.random() < 0.3:
                s += int(rng.integers(1, 5))
            if rng.random() < 0.2:
                d += int(rng.integers(1, 5))
            pieces.append((s, d, ln))
            s += ln
            d += ln
        rng.shuffle(pieces)
        arr = np.array(pieces, dtype=np.uint64).reshape(-1, 3)
        a, sa = kvt_amd.merge_interval(arr)
        b, sb = checkers.oracle_merge(arr)
        assert np.array_equal(a, b) and sa == sb


def test_validate_bounds_known_answers():
    # kvtransfer/tests/send_stub_test.cpp:1141-1158
    assert kvt_amd.validate_bounds([(0, 1024, 512)], 1024, 0, 2)[0] == 0
    assert kvt_amd.validate_bounds([(1, 0, 512)], 1024, 0, 2)[0] == 1
    assert kvt_amd.validate_bounds([(0, 1537, 512)], 2048, 1, 1)[0] == 1
    assert kvt_amd.validate_bounds([(0, 0, 0)], 2048, 1, 1)[0] == 1
    assert kvt_amd.validate_bounds([(0, 0, 8), (0, 2041, 8)], 2048, 1, 1) == (1, 1)
    assert kvt_amd.validate_bounds([(0, 0, 2**63)], 2**64 - 1, 0, 4)[0] == 1
