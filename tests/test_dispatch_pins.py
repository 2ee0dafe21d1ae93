"""What pins the per-destination dispatch (refresh_dst_info, kvtransfer/src/tx_stub.cpp:451-590,
with selection_p_tp, :105-114) of the CPU oracle (kvto_select) and of the product
(kvt_select_parser):

1. a literal table (cache shape, TP relation, equal token sizes) -> (parser, TPKind),
   transcribed row by row from tx_stub.cpp, including the three combinations the reference
   refuses and the engine-TP rule for the shapes that carry linear-attention state;
2. the reference's tests that run THROUGH KvSendStub, i.e. through that dispatch
   (kvtransfer/tests/send_stub_test.cpp:286-496 P16 -> D4, :499-705 P4 -> D16, :707-1130
   P == D): here the ranges are produced from (cache shape, source worker, destination worker)
   alone -- dispatch, then the parser it names, then the merge the test's FakeChannel applies
   -- and must equal the literal triples of those tests, for the oracle and for the product.

The known-answer tests of the individual parsers (test_oracle_known_answers.py,
test_reference_fill_and_indexer_answers.py, test_reference_kda_answers.py) check the same
way that their (workers -> parser, valid ranks, kvt_tp_size, kvt_tp_rank) is what the dispatch
yields (checkers.assert_dispatch).

TPKind has no known answer in the reference's tests (their FakeChannel merges for every
kind); it is pinned by the transcription in (1) alone."""
import numpy as np
import pytest

import checkers
import kvt_amd
from kvt_amd.ctypes_defs import PARSER, TaskBuf, make_worker_info

PEQD, PLTD, PGTD = 0, 1, 2
UNSUPPORTED = None

# (cache shape, relation of the selecting P TP to the D TP, token sizes equal on both sides or
# None = irrelevant) -> (parser, TPKind)                              tx_stub.cpp line
TABLE = [
    (1, "eq", None, "RAGGED_PEQD", PEQD),                             # 475-478
    (1, "gt", True, "RAGGED_PGTD_DPSK", PEQD),                        # 481-483
    (1, "gt", False, "RAGGED_PGTD", PGTD),                            # 484-486
    (1, "lt", None, "RAGGED_PLTD", PLTD),                             # 490-491
    (2, "eq", None, "FLASH_PEQD", PEQD),                              # 495-497
    (2, "gt", None, "FLASH_PGTD", PGTD),                              # 500-502
    (2, "lt", None, UNSUPPORTED, None),                               # falls through to 589
    (3, "eq", None, "HYBRID_PEQD", PEQD),                             # 507-509
    (3, "gt", None, "HYBRID_PGTD", PGTD),                             # 512-514
    (3, "lt", None, "HYBRID_PLTD", PLTD),                             # 517-518
    (4, "eq", None, "DPSK_PEQD", PEQD),                               # 522-524
    (4, "gt", None, "DPSK_PGTD", PEQD),                               # 527-529 (PEQD!)
    (4, "lt", None, "DPSK_PLTD", PEQD),                               # 532-533 (PEQD!)
    (5, "eq", None, "FLASHINFER_PEQD", PEQD),                         # 537-539
    (5, "gt", None, "FLASHINFER_PGTD", PGTD),                         # 542-544
    (5, "lt", None, UNSUPPORTED, None),                               # falls through to 589
    (7, "eq", None, "HYBRID_FI_PEQD", PEQD),                          # 549-551
    (7, "gt", None, "HYBRID_FI_PGTD", PGTD),                          # 554-556
    (7, "lt", None, "HYBRID_FI_PLTD", PLTD),                          # 559-560
    (8, "eq", None, "KIMI_K3_PEQD", PEQD),                            # 564-566
    (8, "gt", None, "KIMI_K3_PGTD", PGTD),                            # 569-571
    (8, "lt", None, "KIMI_K3_PLTD", PLTD),                            # 574-575
    (6, "eq", None, "TURBOQUANT_PEQD", PEQD),                         # 579-581
    (6, "gt", None, "TURBOQUANT_PGTD", PGTD),                         # 584-586
    (6, "lt", None, UNSUPPORTED, None),                               # falls through to 589
]
TP_PAIRS = {"eq": [(1, 1), (4, 4), (16, 16)], "gt": [(2, 1), (4, 2), (16, 4)],
            "lt": [(1, 2), (2, 4), (4, 16)]}


def _workers(p_tp, d_tp, same_tokens, heads=-1, p_rank=0):
    src = make_worker_info([4096 * 16], [4096], 8, tp=p_tp, rank=p_rank, num_kv_heads=heads)
    tok = 4096 if same_tokens else 8192
    dst = make_worker_info([tok * 16], [tok], 8, tp=d_tp, rank=0, num_kv_heads=heads)
    return src, dst


def _select_both(shape, src, dst):
    """-> [(rc, valid, tp_size, tp_rank, parser, kind)] of the oracle and of the product"""
    res = [checkers.oracle_select(shape, src, dst)]
    try:
        res.append((0,) + kvt_amd.select_parser(shape, src, dst))
    except kvt_amd.KvtError as e:
        res.append((e.code, None, None, None, None, None))
    return res


@pytest.mark.parametrize("shape,rel,same,parser,kind", TABLE)
def test_literal_dispatch_table(shape, rel, same, parser, kind):
    for p_tp, d_tp in TP_PAIRS[rel]:
        for same_tokens in ((True, False) if same is None else (same,)):
            for p_rank in {0, p_tp - 1}:
                src, dst = _workers(p_tp, d_tp, same_tokens, p_rank=p_rank)
                for who, got in zip(("oracle", "product"), _select_both(shape, src, dst)):
                    where = (who, shape, p_tp, d_tp, same_tokens, p_rank)
                    if parser is UNSUPPORTED:
                        assert got[0] == 4, where          # "unsupported cache_shape"
                        continue
                    assert got[0] == 0, where
                    # num_kv_heads = -1: every P rank sends (tx_stub.cpp:25-30)
                    assert got[1:4] == ((1 << p_tp) - 1, p_tp, p_rank), where
                    assert got[4:] == (PARSER[parser], kind), where


def test_the_table_names_every_parser_the_dispatch_can_return_exactly_once():
    named = [row[3] for row in TABLE if row[3] is not UNSUPPORTED]
    assert len(named) == len(set(named)) == 22
    # the three KDA state parsers are only ever called by the Kimi-K3 ones
    assert set(PARSER) - set(named) == {"KDA_PEQD", "KDA_PGTD", "KDA_PLTD"}


# selection_p_tp (tx_stub.cpp:105-114): shapes 3, 7 and 8 compare the ENGINE TP of the sender
# with the receiver's, every other shape the number of ranks that really send.
@pytest.mark.parametrize("p_tp,d_tp,heads,valid,p_rank,tp_rank", [
    (8, 2, 2, 0b00010001, 4, 1),      # ComputeValidRanksTest.StridedValidRanks: ranks {0, 4}
    (8, 2, 2, 0b00010001, 3, 1),      # a rank that does not send still counts the ones below it
    (8, 4, 2, 0b01010101, 6, 3),      # send_stub_test.cpp:1803-1807: ranks {0, 2, 4, 6}
])
def test_engine_tp_decides_for_the_shapes_with_linear_attention_state(p_tp, d_tp, heads, valid,
                                                                      p_rank, tp_rank):
    senders = bin(valid).count("1")
    assert senders == d_tp                                  # "equal" by the count of senders
    for shape, by_senders, by_engine in ((1, "RAGGED_PEQD", None), (2, "FLASH_PEQD", None),
                                         (4, "DPSK_PEQD", None), (5, "FLASHINFER_PEQD", None),
                                         (6, "TURBOQUANT_PEQD", None),
                                         (3, None, "HYBRID_PGTD"), (7, None, "HYBRID_FI_PGTD"),
                                         (8, None, "KIMI_K3_PGTD")):
        src, dst = _workers(p_tp, d_tp, False, heads=heads, p_rank=p_rank)
        for who, got in zip(("oracle", "product"), _select_both(shape, src, dst)):
            assert got[:4] == (0, valid, senders, tp_rank), (who, shape)
            if by_engine is None:
                assert got[4:] == (PARSER[by_senders], PEQD), (who, shape)
            else:
                assert got[4:] == (PARSER[by_engine], PGTD), (who, shape)


def test_mixed_regime_p_lt_d_selection():
    # ComputeValidRanksTest.MixedRegimePLtD (send_stub_test.cpp:2739-2745): P tp 2, D tp 8, 4 heads
    for shape, parser in ((1, "RAGGED_PLTD"), (3, "HYBRID_PLTD"), (7, "HYBRID_FI_PLTD"),
                          (4, "DPSK_PLTD"), (8, "KIMI_K3_PLTD")):
        src, dst = _workers(2, 8, False, heads=4, p_rank=1)
        for who, got in zip(("oracle", "product"), _select_both(shape, src, dst)):
            kind = PEQD if shape == 4 else PLTD
            assert got == (0, 0b11, 2, 1, PARSER[parser], kind), (who, shape)


# ----------------------------------------------- the reference's tests through KvSendStub

def _through_the_dispatch(shape, src, dst, tasks):
    """What KvSendStub + the test's FakeChannel deliver for one layer: dispatch, the parser it
    names, then sort-by-source + merge (FakeChannel::register_data merges for every TPKind).
    -> {"oracle": [...], "product": [...]} per-tensor lists of triples, plus the selections."""
    out, picked = {}, {}
    rc, valid, tps, tpr, pid, kind = checkers.oracle_select(shape, src, dst)
    assert rc == 0
    picked["oracle"] = (valid, tps, tpr, pid, kind)
    rc, lists = checkers.oracle_parse(pid, src, dst, valid, tps, tpr, tasks)
    assert rc == 0
    out["oracle"] = [[tuple(int(x) for x in r) for r in checkers.oracle_merge(o)[0]] for o in lists]
    valid, tps, tpr, pid, kind = kvt_amd.select_parser(shape, src, dst)
    picked["product"] = (valid, tps, tpr, pid, kind)
    parser = kvt_amd.Parser(pid, src, dst, valid, tps, tpr)
    bl = kvt_amd.BlockLists()
    for t in tasks:
        assert parser.parse(t.struct, bl) == 0
    out["product"] = [[tuple(int(x) for x in r) for r in kvt_amd.merge_interval(bl.tensor(i))[0]]
                      for i in range(bl.num_tensors())]
    return out, picked


# send_stub_test.cpp:345-475: the 16 messages of one layer, as written there, for P ranks 0 and 1
P16_D4_RANK0 = [(0, 1048576, 512), (512, 1050624, 512), (1024, 1052672, 512), (1536, 1054720, 512),
                (2048, 1056768, 512), (2560, 1058816, 512), (3072, 1060864, 512),
                (3584, 1062912, 512), (4096, 1064960, 512), (4608, 1067008, 512),
                (5120, 1069056, 512), (5632, 1071104, 512), (6144, 1073152, 512),
                (6656, 1075200, 512), (7168, 1077248, 512), (7680, 1079296, 512)]
P16_D4_RANK1 = [(0, 1049088, 512), (512, 1051136, 512), (1024, 1053184, 512), (1536, 1055232, 512),
                (2048, 1057280, 512), (2560, 1059328, 512), (3072, 1061376, 512),
                (3584, 1063424, 512), (4096, 1065472, 512), (4608, 1067520, 512),
                (5120, 1069568, 512), (5632, 1071616, 512), (6144, 1073664, 512),
                (6656, 1075712, 512), (7168, 1077760, 512), (7680, 1079808, 512)]
P16_D4_RANK2_FIRST, P16_D4_RANK3_FIRST = (0, 1049600, 512), (0, 1050112, 512)
P16_D4_RANK2_LAST, P16_D4_RANK3_LAST = (7680, 1080320, 512), (7680, 1080832, 512)


@pytest.mark.parametrize("p_rank", [0, 1, 2, 3])
def test_stub_level_ragged_p16_to_d4(p_rank):
    """ParseBlockSendPGtD (send_stub_test.cpp:286-496): 16 KV heads x 256 x bf16, 64 tokens per
    block; P tp 16 (token 1 KiB), D tp 4 (token 4 KiB); blocks {0,1,2} -> {4,5,6}, 8 tokens."""
    heads, dim, ntpb = 16, 256, 64
    pT, dT = 2 * (heads // 16) * dim * 2, 2 * (heads // 4) * dim * 2
    src = make_worker_info([pT * ntpb], [pT], 8, tp=16, rank=p_rank)
    dst = make_worker_info([dT * ntpb], [dT], 8, tp=4, rank=0)
    out, picked = _through_the_dispatch(1, src, dst, [TaskBuf(0, 8, False, [[0, 1, 2]], [[4, 5, 6]])])
    for who in ("oracle", "product"):
        assert picked[who] == (0xFFFF, 16, p_rank, PARSER["RAGGED_PGTD"], PGTD), who
        got = out[who][0]
        assert len(got) == 16
        if p_rank == 0:
            assert got == P16_D4_RANK0, who
        elif p_rank == 1:
            assert got == P16_D4_RANK1, who
        else:
            first, last = ((P16_D4_RANK2_FIRST, P16_D4_RANK2_LAST) if p_rank == 2 else
                           (P16_D4_RANK3_FIRST, P16_D4_RANK3_LAST))
            assert got[0] == first and got[-1] == last, who
            assert [r[0] for r in got] == [r[0] for r in P16_D4_RANK0], who


# send_stub_test.cpp:553-690: P tp 4 -> D tp 16, D ranks 0 and 1, one layer
P4_D16_RANK0 = [(0, 262144, 512), (2048, 262656, 512), (4096, 263168, 512), (6144, 263680, 512),
                (8192, 264192, 512), (10240, 264704, 512), (12288, 265216, 512),
                (14336, 265728, 512), (16384, 266240, 512), (18432, 266752, 512),
                (20480, 267264, 512), (22528, 267776, 512), (24576, 268288, 512),
                (26624, 268800, 512), (28672, 269312, 512), (30720, 269824, 512)]
P4_D16_RANK1 = [(512, 262144, 512), (2560, 262656, 512), (4608, 263168, 512), (6656, 263680, 512),
                (8704, 264192, 512), (10752, 264704, 512), (12800, 265216, 512),
                (14848, 265728, 512), (16896, 266240, 512), (18944, 266752, 512),
                (20992, 267264, 512), (23040, 267776, 512), (25088, 268288, 512),
                (27136, 268800, 512), (29184, 269312, 512), (31232, 269824, 512)]
P4_D16_RANK2_FIRST, P4_D16_RANK3_FIRST = (1024, 262144, 512), (1536, 262144, 512)


@pytest.mark.parametrize("d_rank", [0, 1, 2, 3])
def test_stub_level_ragged_p4_to_d16(d_rank):
    """ParseBlockSendDGtP (send_stub_test.cpp:499-705): the same model, P tp 4 -> D tp 16."""
    heads, dim, ntpb = 16, 256, 64
    pT, dT = 2 * (heads // 4) * dim * 2, 2 * (heads // 16) * dim * 2
    src = make_worker_info([pT * ntpb], [pT], 8, tp=4, rank=0)
    dst = make_worker_info([dT * ntpb], [dT], 8, tp=16, rank=d_rank)
    out, picked = _through_the_dispatch(1, src, dst, [TaskBuf(0, 8, False, [[0, 1, 2]], [[4, 5, 6]])])
    for who in ("oracle", "product"):
        assert picked[who] == (0xF, 4, 0, PARSER["RAGGED_PLTD"], PLTD), who
        got = out[who][0]
        assert len(got) == 16
        if d_rank == 0:
            assert got == P4_D16_RANK0, who
        elif d_rank == 1:
            assert got == P4_D16_RANK1, who
        else:
            assert got[0] == (P4_D16_RANK2_FIRST if d_rank == 2 else P4_D16_RANK3_FIRST), who
            assert [r[1:] for r in got] == [r[1:] for r in P4_D16_RANK0], who


KB = 1024


def _w16(**kw):
    return make_worker_info([16 * KB], [KB], 16, tp=1, **kw)


def test_stub_level_p_eq_d_for_the_three_shapes_the_reference_runs():
    """ParseBlockSendPEqD (send_stub_test.cpp:707-1130), run by the reference once per value of
    BLLM_KVTRANS_CACHE_SHAPE: B = 16 KiB, T = 1 KiB, 16 blocks, both sides TP 1."""
    B, T = 16 * KB, KB
    first = [TaskBuf(0, 8, False, [[0, 1, 2]], [[4, 5, 6]])]
    # shape 1: one message (0, 4 B, 8 T)                         :790-800
    out, picked = _through_the_dispatch(1, _w16(), _w16(), first)
    for who in out:
        assert picked[who] == (1, 1, 0, PARSER["RAGGED_PEQD"], PEQD)
        assert out[who][0] == [(0, 65536, 8192)]
    # shape 2: K half then V half, V = K + half a layer on each side   :801-818
    out, picked = _through_the_dispatch(2, _w16(), _w16(), first)
    for who in out:
        assert picked[who] == (1, 1, 0, PARSER["FLASH_PEQD"], PEQD)
        assert out[who][0] == [(0, 32768, 4096), (131072, 32768 + 131072, 4096)]
    # shape 3: a chunk that completes no page sends nothing          :760-778
    hybrid_first = [TaskBuf(0, 8, False, [[6], [7], [8], [0, 1, 2]], [[10], [11], [12], [4, 5, 6]])]
    out, picked = _through_the_dispatch(3, _w16(), _w16(), hybrid_first)
    for who in out:
        assert picked[who] == (1, 1, 0, PARSER["HYBRID_PEQD"], PEQD)
        assert out[who][0] == []
    # the second and third sends of the same test                   :830-1128
    out, _ = _through_the_dispatch(1, _w16(), _w16(), [TaskBuf(0, 17, False, [[0, 1, 2]], [[4, 5, 6]])])
    for who in out:
        assert out[who][0] == [(0, 65536, 17408)]
    out, _ = _through_the_dispatch(1, _w16(), _w16(),
                                   [TaskBuf(17, 16, True, [[3, 4, 5]], [[7, 8, 9]])])
    for who in out:
        assert out[who][0] == [(4 * B + T, 8 * B + T, 16 * T)]
    out, _ = _through_the_dispatch(
        3, _w16(), _w16(), [TaskBuf(17, 16, True, [[6], [7], [8], [3, 4, 5]],
                                    [[10], [11], [12], [7, 8, 9]])])
    for who in out:
        assert out[who][0] == [(4 * B, 8 * B, 5 * B)]
    out, _ = _through_the_dispatch(
        3, _w16(), _w16(), [TaskBuf(1, 3, True, [[4], [5], [6], [3]], [[8], [9], [10], [7]])])
    for who in out:
        assert out[who][0] == [(3 * B, 7 * B, 4 * B)]


def test_swapping_two_table_rows_is_noticed():
    """The literal table is not a tautology: exchanging the answers of two rows makes the
    comparison of test_literal_dispatch_table fail for both implementations."""
    swapped = list(TABLE)
    swapped[4], swapped[5] = (TABLE[4][:3] + TABLE[5][3:]), (TABLE[5][:3] + TABLE[4][3:])
    mismatches = 0
    for shape, rel, same, parser, kind in swapped[4:6]:
        p_tp, d_tp = TP_PAIRS[rel][1]
        src, dst = _workers(p_tp, d_tp, True)
        for got in _select_both(shape, src, dst):
            mismatches += got[4:] != (PARSER[parser], kind)
    assert mismatches == 4
