"""The CPU oracle against golden vectors written by the compiled reference.

tests/golden/parse_golden.json is produced by tests/golden/make_golden.py from
the reference's own ParseBlock sources; this test needs neither the reference
nor oracle/_ref at run time.
"""
import json
import os

import numpy as np
import pytest

import cases
import checkers

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "parse_golden.json")
with open(GOLDEN) as f:
    _CASES = json.load(f)


def test_fixture_is_substantial():
    assert len(_CASES) >= 120
    assert sum(len(t) for c in _CASES for t in c["expect"]) > 5000
    assert {c["parser"] for c in _CASES} >= set(cases.ALL_PARSERS)


@pytest.mark.parametrize("case", _CASES, ids=[c["name"] for c in _CASES])
def test_oracle_matches_golden(case):
    pid, src, dst, valid, tps, tpr, tasks = cases.materialise(case)
    rc, outs = checkers.oracle_parse(pid, src, dst, valid, tps, tpr, tasks, fp8=case["fp8"])
    assert rc == case["rc"]
    if rc != 0:
        return
    assert len(outs) == len(case["expect"])
    for got, exp in zip(outs, case["expect"]):
        exp = np.array(exp, dtype=np.uint64).reshape(-1, 3)
        assert np.array_equal(got, exp)
