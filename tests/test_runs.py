"""Strided runs: kvt_parse_block_runs must describe exactly the range sequence
of kvt_parse_block (which test_parse_parity.py pins against the oracle and the
reference's golden vectors), for every parser; kvt_run_lists_compress must be
an exact inverse of expansion. CPU only."""
import json
import os

import numpy as np
import pytest

import cases
import checkers
import kvt_amd
from test_parse_parity import _same, product_parse

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "parse_golden.json")
with open(GOLDEN) as f:
    _GOLDEN = json.load(f)


def numpy_expand(runs):
    """Independent expansion of a structured kvt_run array -> (n,3) uint64."""
    out = []
    for r in runs:
        n0, n1, n2 = (int(v) for v in r["n"])
        ss, ds = [int(v) for v in r["src_stride"]], [int(v) for v in r["dst_stride"]]
        for a in range(n0):
            for b in range(n1):
                for c in range(n2):
                    out.append((int(r["src_offset"]) + a * ss[0] + b * ss[1] + c * ss[2],
                                int(r["dst_offset"]) + a * ds[0] + b * ds[1] + c * ds[2],
                                int(r["length"])))
    return np.asarray(out, dtype=np.uint64).reshape(-1, 3)


def product_parse_runs(case, pad=True):
    pid, src, dst, valid, tps, tpr, tasks = cases.materialise(case)
    parser = kvt_amd.Parser(pid, src, dst, valid, tps, tpr, fp8=case["fp8"], pad=pad)
    runs = kvt_amd.RunLists()
    for t in tasks:
        rc = parser.parse_runs(t.struct, runs)
        if rc != 0:
            return rc, None
    return 0, runs


@pytest.mark.parametrize("case", _GOLDEN, ids=[c["name"] for c in _GOLDEN])
def test_runs_expand_to_the_reference_golden_lists(case):
    rc, runs = product_parse_runs(case)
    assert rc == case["rc"]
    if rc == 0:
        _same(runs.expand().all(), case["expect"], case["name"])
        _same([numpy_expand(runs.tensor(t)) for t in range(runs.num_tensors())], case["expect"],
              case["name"])


@pytest.mark.parametrize("parser", cases.ALL_PARSERS)
def test_runs_expand_to_the_plain_lists_on_random_cases(parser):
    n_runs = n_ranges = 0
    for seed in range(200, 400):
        case = cases.gen_case(parser, seed)
        rc_p, out_p = product_parse(case)
        rc_r, runs = product_parse_runs(case)
        assert rc_r == rc_p, case["name"]
        if rc_p != 0:
            continue
        _same(runs.expand().all(), out_p, case["name"])
        for t in range(runs.num_tensors()):
            ranges, nbytes = runs.totals(t)
            assert ranges == len(out_p[t]) and nbytes == int(out_p[t][:, 2].sum())
            n_runs += len(runs.tensor(t))
            n_ranges += ranges
    assert 0 < n_runs <= n_ranges
    if parser in ("FLASH_PGTD", "RAGGED_PGTD", "RAGGED_PLTD", "FLASHINFER_PGTD", "FLASHINFER_PLTD"):
        assert n_runs * 2 < n_ranges      # per-token parsers really fold


@pytest.mark.parametrize("parser", ["RAGGED_PGTD", "FLASH_PGTD", "DPSK_PLTD"])
def test_runs_with_fp8_lengths(parser):
    for seed in range(500, 540):
        case = cases.gen_case(parser, seed)
        case["fp8"] = True
        rc_p, out_p = product_parse(case)
        rc_r, runs = product_parse_runs(case)
        assert rc_r == rc_p
        if rc_p == 0:
            _same(runs.expand().all(), out_p, case["name"])


@pytest.mark.parametrize("parser", cases.ALL_PARSERS)
def test_compress_is_the_exact_inverse_of_expansion(parser):
    folded = total = 0
    for seed in range(700, 760):
        case = cases.gen_case(parser, seed)
        pid, src, dst, valid, tps, tpr, tasks = cases.materialise(case)
        rc, outs = checkers.oracle_parse(pid, src, dst, valid, tps, tpr, tasks)
        if rc != 0:
            continue
        lists = kvt_amd.BlockLists()
        for t, o in enumerate(outs):
            lists.append(t, o)
        runs = kvt_amd.RunLists.compress(lists)
        _same(runs.expand().all(), outs, case["name"])
        _same([numpy_expand(runs.tensor(t)) for t in range(runs.num_tensors())], outs,
              case["name"])
        folded += sum(len(runs.tensor(t)) for t in range(runs.num_tensors()))
        total += sum(len(o) for o in outs)
    assert folded <= total


def test_compress_on_hand_made_lists():
    B = kvt_amd.BlockLists()
    # K,V interleaved per token, 3 tokens, then an unrelated range, then a descending pair
    rows = []
    for tok in range(3):
        rows += [(1000 + tok * 64, 5000 + tok * 256, 32), (1000 + tok * 64 + 4096, 5000 + tok * 256 + 128, 32)]
    rows += [(9000, 100, 48), (800, 90000, 16), (700, 90016, 16)]
    B.append(0, rows)
    R = kvt_amd.RunLists.compress(B)
    runs = R.tensor(0)
    assert len(runs) == 4
    assert runs[0]["n"].tolist() == [1, 3, 2]
    assert runs[0]["src_stride"].tolist() == [0, 64, 4096]
    assert runs[0]["dst_stride"].tolist() == [0, 256, 128]
    assert [r["n"].tolist() for r in runs[1:]] == [[1, 1, 1]] * 3   # no negative strides
    assert np.array_equal(R.expand().tensor(0), np.asarray(rows, np.uint64))
    assert R.totals(0) == (9, 6 * 32 + 48 + 32)


def test_empty_and_error_cases():
    R = kvt_amd.RunLists()
    assert R.num_tensors() == 0
    assert kvt_amd.RunLists.compress(kvt_amd.BlockLists()).num_tensors() == 0
    L = kvt_amd.lib()
    assert L.kvt_run_lists_expand(None, None) == kvt_amd.ctypes_defs.ERR_INVALID
    assert L.kvt_parse_block_runs(None, None, None) == kvt_amd.ctypes_defs.ERR_INVALID
