"""The CPU oracle against the compiled reference (oracle/_ref), range for range.

Skipped where oracle/_ref was never built (it needs the reference checkout).
"""
import numpy as np
import pytest

import cases
import checkers

pytestmark = pytest.mark.skipif(checkers.ref() is None, reason="oracle/_ref not built")


def _compare(case):
    pid, src, dst, valid, tps, tpr, tasks = cases.materialise(case)
    rc_r, out_r = checkers.ref_parse(pid, src, dst, valid, tps, tpr, tasks)
    rc_o, out_o = checkers.oracle_parse(pid, src, dst, valid, tps, tpr, tasks, fp8=case["fp8"])
    assert rc_r == rc_o, case["name"]
    assert len(out_r) == len(out_o), case["name"]
    for t, (a, b) in enumerate(zip(out_r, out_o)):
        assert a.shape == b.shape, (case["name"], t, a.shape, b.shape)
        assert np.array_equal(a, b), (case["name"], t)
    return sum(len(a) for a in out_r)


@pytest.mark.parametrize("parser", cases.ALL_PARSERS)
def test_random_cases_match_reference(parser):
    emitted = 0
    for seed in range(150):
        emitted += _compare(cases.gen_case(parser, seed))
    assert emitted > 0


@pytest.mark.parametrize("parser", ["RAGGED_PEQD", "FLASH_PEQD", "DPSK_PEQD", "FLASHINFER_PEQD",
                                    "HYBRID_PEQD", "RAGGED_PGTD", "FLASH_PGTD"])
def test_out_of_pool_block_id_is_rejected_like_reference(parser):
    hits = 0
    for seed in range(40):
        case = cases.gen_case(parser, 1000 + seed)
        # push one destination block id beyond the destination pool
        t = case["tasks"][0]
        g = len(t[4]) - 1
        while g >= 0 and not t[4][g]:
            g -= 1
        t[4][g][0] = case["dst"]["layer_num_blocks"] + 3
        pid, src, dst, valid, tps, tpr, tasks = cases.materialise(case)
        rc_r, _ = checkers.ref_parse(pid, src, dst, valid, tps, tpr, tasks)
        rc_o, _ = checkers.oracle_parse(pid, src, dst, valid, tps, tpr, tasks)
        assert rc_r == rc_o, case["name"]
        hits += rc_r != 0
    assert hits > 0
