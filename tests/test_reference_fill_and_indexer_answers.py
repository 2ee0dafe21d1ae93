"""More of the numbers the reference's own unit tests assert, for the hybrid P > D parsers:
the indexer that only a representative rank sends, the zero fill of the receiver's last
block, and the replicated-head FlashInfer case (kvtransfer/tests/send_stub_test.cpp; line
ranges cited per test). Every expectation is checked against the CPU oracle and against the
product parser through the C ABI."""
import pytest

import checkers
import kvt_amd
from kvt_amd.ctypes_defs import PARSER, TaskBuf, make_worker_info


def _both(parser, src, dst, task, heads):
    """-> the list both implementations produce for one task (they must agree)."""
    valid = checkers.oracle().kvto_valid_ranks(src.engine_tp_size, dst.engine_tp_size, heads)
    tp_size = bin(valid).count("1")
    tp_rank = bin(valid & ((1 << src.worker_tp_rank) - 1)).count("1")
    checkers.assert_dispatch(parser, src, dst, valid, tp_size, tp_rank)
    rc, outs = checkers.oracle_parse(PARSER[parser], src, dst, valid, tp_size, tp_rank, [task])
    assert rc == 0 and len(outs) == 1
    oracle = [tuple(int(x) for x in r) for r in outs[0]]
    p = kvt_amd.Parser(PARSER[parser], src, dst, valid, tp_size, tp_rank)
    lists = kvt_amd.BlockLists()
    assert p.parse(task.struct, lists) == 0
    product = [tuple(int(x) for x in r) for r in lists.tensor(0)] if lists.num_tensors() else []
    assert product == oracle
    return oracle


# make_qwen3_next_flash_pgtd_workers, send_stub_test.cpp:1841-1883: 8 KV heads x 128 x bf16,
# 16 tokens per block, P tp 4 -> D tp 2, one GDN layer with conv {1,3,4} / ssm {1,1,2,2} x 1 B
def _flash_workers(p_rank=0, **extra):
    kw = dict(num_kv_heads=8, num_gdn_layers=1, conv_state_shape=[1, 3, 4],
              ssm_state_shape=[1, 1, 2, 2], gdn_conv_channel_dims=[2, 2], attn_kernel_blk_ntpb=16)
    kw.update(extra)
    pT, dT = 2 * 2 * 128 * 2, 2 * 4 * 128 * 2
    idx = {k: kw.pop(k) for k in ("p_indexer", "d_indexer") if k in kw}
    src = make_worker_info([pT * 16], [pT], 256, tp=4, rank=p_rank,
                           indexer_blk_ntpb=idx.get("p_indexer", 0), **kw)
    dst = make_worker_info([dT * 16], [dT], 256, tp=2, rank=p_rank // 2,
                           indexer_blk_ntpb=idx.get("d_indexer", 0), **kw)
    return src, dst


# make_qwen3_next_flashinfer_pgtd_workers, send_stub_test.cpp:2058-2096: 4 KV heads x 64 x bf16
def _flashinfer_workers(p_rank=0, **extra):
    kw = dict(num_kv_heads=4, num_gdn_layers=1, conv_state_shape=[1, 3, 4],
              ssm_state_shape=[1, 1, 2, 2], gdn_conv_channel_dims=[2, 2], attn_kernel_blk_ntpb=16)
    kw.update(extra)
    pT, dT = 2 * 1 * 64 * 2, 2 * 2 * 64 * 2
    idx = {k: kw.pop(k) for k in ("p_indexer", "d_indexer") if k in kw}
    src = make_worker_info([pT * 16], [pT], 256, tp=4, rank=p_rank,
                           indexer_blk_ntpb=idx.get("p_indexer", 0), **kw)
    dst = make_worker_info([dT * 16], [dT], 256, tp=2, rank=p_rank // 2,
                           indexer_blk_ntpb=idx.get("d_indexer", 0), **kw)
    return src, dst


# send_stub_test.cpp:1887-1946 and :2100-2157: P ranks 0/1 feed D rank 0, 2/3 feed D rank 1; the
# first rank of each pair sends the replicated indexer cache, the other one does not
@pytest.mark.parametrize("parser,workers,heads", [("HYBRID_PGTD", _flash_workers, 8),
                                                  ("HYBRID_FI_PGTD", _flashinfer_workers, 4)])
def test_indexer_is_sent_by_the_representative_rank_of_each_d_rank(parser, workers, heads):
    task = TaskBuf(1, 5, False, [[100], [30, 31], [0]], [[200], [40], [10]])
    idx = dict(p_indexer=4, d_indexer=8, hybrid_indexer_token_size=32)
    src, dst = workers(2, **idx)
    rep = _both(parser, src, dst, task, heads)
    pB, dB = int(src.block_sizes[0]), int(dst.block_sizes[0])
    assert rep[0] == (30 * pB + 1 * 32, 40 * dB + 1 * 32, 3 * 32)
    assert rep[1] == (31 * pB, 40 * dB + 4 * 32, 2 * 32)
    src, dst = workers(1, **idx)
    nonrep = _both(parser, src, dst, task, heads)
    assert len(nonrep) + 2 == len(rep)
    assert (30 * pB + 32, 40 * dB + 32, 96) not in nonrep


# send_stub_test.cpp:1948-2001
def test_flash_p_gt_d_fills_the_tail_of_the_last_decode_block():
    src, dst = _flash_workers()
    pB, dB = int(src.block_sizes[0]), int(dst.block_sizes[0])
    p_step, d_step = int(src.token_sizes[0]) // 2, int(dst.token_sizes[0]) // 2
    o = _both("HYBRID_PGTD", src, dst,
              TaskBuf(5, 18, True, [[100, 101], [0, 1, 2]], [[200, 201], [10, 11, 12]]), 8)
    filled, to_fill = 23 % 16, 16 - 23 % 16                     # 7 filled, 9 to fill
    assert len(o) == 14 + 36 + to_fill * 2                      # GDN, attention, fill
    fk, fv = o[-to_fill * 2], o[-to_fill * 2 + 1]
    d_kernel_half = 16 * int(dst.token_sizes[0]) // 2
    assert fk == (0, 11 * dB + filled * d_step, p_step)
    assert fv == (0, 11 * dB + filled * d_step + d_kernel_half, p_step)
    assert pB == 16 * 2 * p_step


# send_stub_test.cpp:2003-2027 and :2029-2054
def test_flash_p_gt_d_no_fill_when_aligned_or_not_the_last_chunk():
    src, dst = _flash_workers()
    groups = ([[100, 101], [0, 1, 2]], [[200, 201], [10, 11, 12]])
    assert len(_both("HYBRID_PGTD", src, dst, TaskBuf(0, 16, True, *groups), 8)) == 14 + 32
    assert len(_both("HYBRID_PGTD", src, dst, TaskBuf(5, 18, False, *groups), 8)) == 36


# send_stub_test.cpp:2159-2220
def test_flashinfer_p_gt_d_fills_the_tail_of_the_last_decode_block():
    src, dst = _flashinfer_workers()
    dB, dT = int(dst.block_sizes[0]), int(dst.token_sizes[0])
    heads_per_rank = 4 // 4
    head_row = int(src.token_sizes[0]) // 2 // heads_per_rank
    o = _both("HYBRID_FI_PGTD", src, dst,
              TaskBuf(0, 20, True, [[100], [0, 1]], [[200], [10, 11]]), 4)
    filled, to_fill = 20 % 16, 16 - 20 % 16                     # 4 filled, 12 to fill
    fill_records = heads_per_rank * 2
    assert len(o) == 7 + heads_per_rank * 2 * 2 + fill_records
    fk, fv = o[-fill_records], o[-fill_records + 1]
    assert fk == (0, 11 * dB + filled * head_row, to_fill * head_row)
    assert fv == (0, 11 * dB + filled * head_row + 16 * dT // 2, to_fill * head_row)


# send_stub_test.cpp:2222-2249 and :2251-2278
def test_flashinfer_p_gt_d_no_fill_when_aligned_or_not_the_last_chunk():
    src, dst = _flashinfer_workers()
    groups = ([[100], [0, 1]], [[200], [10, 11]])
    assert len(_both("HYBRID_FI_PGTD", src, dst, TaskBuf(0, 16, True, *groups), 4)) == 7 + 2
    assert len(_both("HYBRID_FI_PGTD", src, dst, TaskBuf(0, 20, False, *groups), 4)) == 2 * 2


# send_stub_test.cpp:1757-1831: 2 KV heads in total on P tp 4 -> every rank holds one physical
# head; only ranks 0 and 2 send, and the head is not split in two
def test_flashinfer_p_gt_d_replicated_kv_heads_partial_block():
    kw = dict(num_kv_heads=2, num_gdn_layers=1, attn_kernel_blk_ntpb=16)
    T = 2 * 1 * 64 * 2
    src = make_worker_info([T * 16], [T], 256, tp=4, rank=0, **kw)
    dst = make_worker_info([T * 16], [T], 256, tp=2, rank=0, **kw)
    assert checkers.oracle().kvto_valid_ranks(4, 2, 2) == 0b0101
    o = _both("HYBRID_FI_PGTD", src, dst, TaskBuf(0, 5, False, [[100], [0]], [[200], [10]]), 2)
    B = T * 16
    assert o == [(0, 10 * B, 5 * 128), (B // 2, 10 * B + B // 2, 5 * 128)]


# ---------------------------------------------------------------- P < D (p_tp 2 -> d_tp 8)

# make_qwen3_next_flash_pltd_workers / ..._flashinfer_..., send_stub_test.cpp:2334-2398:
# kv_heads 2 = replicated rows, kv_heads 4 = mixed (P row = 2 x D row); conv {1,3,8},
# ssm {1,1,2,4}, channel dims {4,4}, 1-byte elements
def _pltd_workers(kv_heads, d_rank, head_dim, **src_extra):
    kw = dict(num_kv_heads=kv_heads, num_gdn_layers=1, conv_state_shape=[1, 3, 8],
              ssm_state_shape=[1, 1, 2, 4], gdn_conv_channel_dims=[4, 4], attn_kernel_blk_ntpb=16)
    pT = 2 * max(1, kv_heads // 2) * head_dim * 2
    dT = 2 * max(1, kv_heads // 8) * head_dim * 2
    src = make_worker_info([pT * 16], [pT], 256, tp=2, rank=0, **kw, **src_extra)
    dst = make_worker_info([dT * 16], [dT], 256, tp=8, rank=d_rank, **kw)
    return src, dst


def _pltd(parser, src, dst, task, heads):
    """The reference's P<D tests call the parser with kvt_tp_size 2, kvt_tp_rank 0."""
    valid = checkers.oracle().kvto_valid_ranks(2, 8, heads)
    assert bin(valid).count("1") == 2
    checkers.assert_dispatch(parser, src, dst, valid, 2, 0)
    rc, outs = checkers.oracle_parse(PARSER[parser], src, dst, valid, 2, 0, [task])
    assert rc == 0 and len(outs) == 1
    oracle = [tuple(int(x) for x in r) for r in outs[0]]
    p = kvt_amd.Parser(PARSER[parser], src, dst, valid, 2, 0)
    lists = kvt_amd.BlockLists()
    assert p.parse(task.struct, lists) == 0
    assert [tuple(int(x) for x in r) for r in lists.tensor(0)] == oracle
    return oracle


ONE_BLOCK = ([[100], [1]], [[200], [10]])


# send_stub_test.cpp:2402-2434
def test_flash_p_lt_d_replicated_rows_copy_the_full_block():
    src, dst = _pltd_workers(2, 1, 128)
    o = _pltd("HYBRID_PLTD", src, dst, TaskBuf(0, 16, True, *ONE_BLOCK), 2)
    pB = int(src.block_sizes[0])
    assert len(o) == 1 + 7 and o[0] == (1 * pB, 10 * pB, pB)


# send_stub_test.cpp:2436-2498: D ranks 0/1 take head 0 of P rank 0, D ranks 2/3 head 1
def test_flash_p_lt_d_mixed_regime_takes_one_head_slice():
    src, dst = _pltd_workers(4, 2, 128)
    o = _pltd("HYBRID_PLTD", src, dst, TaskBuf(0, 5, False, *ONE_BLOCK), 4)
    pB, dB = int(src.block_sizes[0]), int(dst.block_sizes[0])
    p_step, d_step = int(src.token_sizes[0]) // 2, int(dst.token_sizes[0]) // 2
    assert (pB, dB, p_step, d_step) == (16 * 1024, 16 * 512, 512, 256)
    assert len(o) == 10
    for t in range(5):
        k, v = o[2 * t], o[2 * t + 1]
        assert k == (1 * pB + t * p_step + 1 * d_step, 10 * dB + t * d_step, d_step)
        assert v == (k[0] + pB // 2, k[1] + dB // 2, d_step)
    src0, dst0 = _pltd_workers(4, 1, 128)
    o0 = _pltd("HYBRID_PLTD", src0, dst0, TaskBuf(0, 5, False, *ONE_BLOCK), 4)
    assert len(o0) == 10 and o0[0][:2] == (1 * pB, 10 * dB)


# send_stub_test.cpp:2500-2547
def test_flash_p_lt_d_mixed_regime_fills_the_tail_and_slices_the_gdn_state():
    src, dst = _pltd_workers(4, 2, 128)
    o = _pltd("HYBRID_PLTD", src, dst, TaskBuf(0, 5, True, *ONE_BLOCK), 4)
    pB, dB = int(src.block_sizes[0]), int(dst.block_sizes[0])
    d_step = int(dst.token_sizes[0]) // 2
    assert len(o) == 10 + 2 + 7
    assert o[10] == (1 * pB, 10 * dB + 5 * d_step, 11 * d_step)
    assert o[11] == (1 * pB, 10 * dB + 5 * d_step + dB // 2, 11 * d_step)
    # gdn_group_n 4, gdn_group_off 2 for D rank 2: per-channel slice of 4 / 4 = 1 byte
    assert o[12] == (100 * pB + 2 * 1, 200 * dB, 1)


# send_stub_test.cpp:2549-2602
def test_flashinfer_p_lt_d_mixed_regime_takes_one_head_section():
    src, dst = _pltd_workers(4, 2, 64)
    o = _pltd("HYBRID_FI_PLTD", src, dst, TaskBuf(0, 5, False, *ONE_BLOCK), 4)
    pB, dB = int(src.block_sizes[0]), int(dst.block_sizes[0])
    row = int(dst.token_sizes[0]) // 2
    assert (pB, dB, row) == (16 * 512, 16 * 256, 128)
    assert o == [(1 * pB + 1 * 16 * row, 10 * dB, 5 * row),
                 (1 * pB + 1 * 16 * row + pB // 2, 10 * dB + dB // 2, 5 * row)]
    src0, dst0 = _pltd_workers(4, 1, 64)
    o0 = _pltd("HYBRID_FI_PLTD", src0, dst0, TaskBuf(0, 5, False, *ONE_BLOCK), 4)
    assert len(o0) == 2 and o0[0][0] == 1 * pB


# send_stub_test.cpp:2604-2644
def test_flashinfer_p_lt_d_mixed_regime_fills_the_tail():
    src, dst = _pltd_workers(4, 2, 64)
    o = _pltd("HYBRID_FI_PLTD", src, dst, TaskBuf(0, 5, True, *ONE_BLOCK), 4)
    pB, dB = int(src.block_sizes[0]), int(dst.block_sizes[0])
    row = int(dst.token_sizes[0]) // 2
    assert len(o) == 2 + 2 + 7
    assert o[2] == (1 * pB, 10 * dB + 5 * row, 11 * row)
    assert o[3] == (1 * pB, 10 * dB + 5 * row + dB // 2, 11 * row)


# ------------------------------------------------------------- PLE state (replicated)

PLE = dict(num_ple_layers=1, ple_block_group=2, ple_conv_state_shape=[256, 3, 4],
           ple_conv_elem_size=2)
PLE_GROUPS = ([[100], [1], [150]], [[200], [10], [220]])


# send_stub_test.cpp:2646-2695: P ranks 0/1 both feed D rank 0; rank 0 alone sends the
# replicated PLE state (3 x 4 x 2 bytes)
@pytest.mark.parametrize("p_rank,expected", [(0, 1), (1, 0)])
def test_ple_state_p_gt_d_is_sent_once_by_the_representative_rank(p_rank, expected):
    src, dst = _flash_workers(p_rank)
    src = make_worker_info([int(src.block_sizes[0])], [int(src.token_sizes[0])], 256, tp=4,
                           rank=p_rank, num_kv_heads=8, num_gdn_layers=1,
                           conv_state_shape=[1, 3, 4], ssm_state_shape=[1, 1, 2, 2],
                           gdn_conv_channel_dims=[2, 2], attn_kernel_blk_ntpb=16, **PLE)
    o = _both("HYBRID_PGTD", src, dst, TaskBuf(0, 1, True, *PLE_GROUPS), 8)
    want = (150 * int(src.block_sizes[0]), 220 * int(dst.block_sizes[0]), 3 * 4 * 2)
    assert o.count(want) == expected


# send_stub_test.cpp:2697-2737: every D rank receives the complete state
@pytest.mark.parametrize("d_rank", [0, 3])
def test_ple_state_p_lt_d_fans_out_complete(d_rank):
    src, dst = _pltd_workers(4, d_rank, 128, **PLE)
    o = _pltd("HYBRID_PLTD", src, dst, TaskBuf(0, 1, True, *PLE_GROUPS), 4)
    want = (150 * int(src.block_sizes[0]), 220 * int(dst.block_sizes[0]), 3 * 4 * 2)
    assert o.count(want) == 1


# send_stub_test.cpp:23-41 (Qwen4PleParseBlockTest.PEqDCopiesFullPaddedBlock calls the PLE helper
# directly: 64-byte pages, PLE block group 2, block 2 -> 5): the same record through the
# top-level P == D parser with empty GDN and attention groups
def test_ple_state_p_eq_d_copies_the_full_padded_page():
    kw = dict(num_gdn_layers=1, num_kv_heads=1, **PLE)
    w = make_worker_info([64], [64], 16, tp=1, rank=0, **kw)
    o = _both("HYBRID_PEQD", w, w, TaskBuf(0, 0, True, [[], [], [2]], [[], [], [5]]), 1)
    assert o == [(2 * 64, 5 * 64, 64)]
