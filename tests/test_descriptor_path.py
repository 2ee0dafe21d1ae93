"""The product parser against the reference's SECOND statement of the byte mapping.

Besides the hand-written ParseBlock functions the reference carries a
descriptor-driven generator (build_transfer_plan + generate_all_ipc_blocks,
kvtransfer/src/cache_transfer_spec.cpp:293-307, 616-848): a closed form
``block * block_stride + token * token_stride + base + head * head_stride`` that
emits one range per token. Nothing in the reference calls it, but it is an
independent derivation of which source byte lands on which destination byte, so
it pins the product from a second side: after both lists are brought to the same
normal form (sorted by destination, maximal runs), they must be identical.

Where the two reference implementations agree with each other this holds for
the product too: RAGGED_FLASH, FLASH and DPSK_V32 cache shapes, P==D and P>D.
For FLASHINFER and QWEN3_NEXT the descriptor path describes a different mapping
than the parsers the reference actually dispatches (it writes V without a head
stride and has no notion of trailing pages, pack size or PLE groups), so those
shapes stay pinned by the hand-written parsers only.

Skipped where oracle/_ref was never built (it needs the reference checkout).
"""
import numpy as np
import pytest

import cases
import checkers
import kvt_amd
from kvt_amd.ctypes_defs import (SHAPE_DPSK_V32_SPARSE_MLA, SHAPE_FLASH, SHAPE_RAGGED_FLASH)

pytestmark = pytest.mark.skipif(checkers.ref() is None, reason="oracle/_ref not built")

FAMILIES = {
    "RAGGED_PEQD": SHAPE_RAGGED_FLASH, "RAGGED_PGTD": SHAPE_RAGGED_FLASH,
    "RAGGED_PGTD_DPSK": SHAPE_RAGGED_FLASH,
    "FLASH_PEQD": SHAPE_FLASH, "FLASH_PGTD": SHAPE_FLASH,
    "DPSK_PEQD": SHAPE_DPSK_V32_SPARSE_MLA, "DPSK_PGTD": SHAPE_DPSK_V32_SPARSE_MLA,
}


def normal_form(ranges):
    """Sorted by destination with touching ranges joined: two lists that move the same
    bytes to the same places have the same normal form as long as no destination byte is
    written twice (true within one request)."""
    a = ranges[ranges[:, 2] > 0]
    if len(a) == 0:
        return a.reshape(0, 3)
    a = a[np.lexsort((a[:, 0], a[:, 1]))]
    joins = (a[:-1, 0] + a[:-1, 2] == a[1:, 0]) & (a[:-1, 1] + a[:-1, 2] == a[1:, 1])
    starts = np.concatenate(([True], ~joins))
    group = np.cumsum(starts) - 1
    out = a[starts].copy()
    out[:, 2] = np.bincount(group, weights=a[:, 2].astype(np.float64)).astype(np.uint64)
    return out


def _adapt(case):
    """The descriptor path reads fields the hand-written parsers ignore for these shapes:
    it treats num_gdn_layers > 0 as a hybrid cache, and takes tensor t's block ids from
    block group t where the DPSK parsers use group 0 for every tensor."""
    case["src"]["num_gdn_layers"] = 0
    case["dst"]["num_gdn_layers"] = 0
    if case["parser"].startswith("DPSK"):
        for t in case["tasks"]:
            t[3] = [t[3][0], t[3][0]]
            t[4] = [t[4][0], t[4][0]]
    return case


@pytest.mark.parametrize("parser", sorted(FAMILIES))
def test_product_moves_the_bytes_the_descriptor_path_describes(parser):
    compared = moved = 0
    for seed in range(120):
        case = _adapt(cases.gen_case(parser, seed))
        pid, src, dst, valid, tps, tpr, tasks = cases.materialise(case)
        product = kvt_amd.Parser(pid, src, dst, valid, tps, tpr)
        for task in tasks:                       # one request at a time: see normal_form
            lists = kvt_amd.BlockLists()
            assert product.parse(task.struct, lists) == 0, case["name"]
            got = lists.all()
            rc, want, _ = checkers.ref_plan_parse(FAMILIES[parser], src, dst, valid, tps, tpr,
                                                  [task])
            assert rc == 0, case["name"]
            for t in range(max(len(got), len(want))):
                a = normal_form(got[t]) if t < len(got) else np.zeros((0, 3), np.uint64)
                b = normal_form(want[t]) if t < len(want) else np.zeros((0, 3), np.uint64)
                assert a.shape == b.shape and np.array_equal(a, b), (case["name"], t)
                moved += int(a[:, 2].sum())
            compared += 1
    assert compared >= 120 and moved > 0


def test_normal_form_joins_only_what_touches_on_both_sides():
    r = np.array([[64, 0, 16], [0, 32, 16], [80, 16, 16], [16, 48, 8], [100, 56, 8]], np.uint64)
    assert normal_form(r).tolist() == [[64, 0, 32], [0, 32, 24], [100, 56, 8]]
