"""Known-answer checks of the CPU oracle.

The expectations are the numbers the reference's own unit tests assert
(kvtransfer/tests/send_stub_test.cpp; line ranges cited per test) and the
closed forms of each layout, restated here as data.
"""
import numpy as np
import pytest

import checkers
from kvt_amd.ctypes_defs import PARSER, TaskBuf, make_worker_info

KB = 1024


def _parse(parser, src, dst, tasks, valid=None, tp_size=None, tp_rank=None, dispatch=True, **kw):
    valid = (1 << src.engine_tp_size) - 1 if valid is None else valid
    tp_size = bin(valid).count("1") if tp_size is None else tp_size
    tp_rank = bin(valid & ((1 << src.worker_tp_rank) - 1)).count("1") if tp_rank is None else tp_rank
    if dispatch:   # the case reaches this parser, with these ranks, through the dispatch too
        checkers.assert_dispatch(parser, src, dst, valid, tp_size, tp_rank)
    rc, outs = checkers.oracle_parse(PARSER[parser], src, dst, valid, tp_size, tp_rank, tasks, **kw)
    assert rc == 0
    return [[tuple(int(x) for x in r) for r in o] for o in outs]


def _sorted_by_src(rows):
    return sorted(rows, key=lambda r: r[0])


# send_stub_test.cpp:286-496 (ParseBlockSendPGtD): 16 heads x 256 x bf16, 64 tokens
# per block, P tp 16 -> D tp 4, first 8 tokens of blocks {0,1,2} -> {4,5,6}.
@pytest.mark.parametrize("p_rank", [0, 1, 2, 3, 5, 15])
def test_ragged_p_gt_d_known_answer(p_rank):
    src = make_worker_info([1024 * 64], [1024], 8, tp=16, rank=p_rank)
    dst = make_worker_info([4096 * 64], [4096], 8, tp=4, rank=p_rank // 4)
    out = _parse("RAGGED_PGTD", src, dst, [TaskBuf(0, 8, False, [[0, 1, 2]], [[4, 5, 6]])])
    goff = p_rank % 4
    exp = []
    for t in range(8):
        exp.append((1024 * t, 1048576 + 4096 * t + 512 * goff, 512))
        exp.append((1024 * t + 512, 1048576 + 4096 * t + 2048 + 512 * goff, 512))
    assert _sorted_by_src(out[0]) == exp
    # emission order: all K records of the task, then all V records
    assert out[0][:8] == exp[0::2] and out[0][8:] == exp[1::2]


def test_ragged_p_gt_d_first_values_literal():
    # literal numbers asserted at send_stub_test.cpp:346-378 for p_rank 0
    src = make_worker_info([65536], [1024], 8, tp=16, rank=0)
    dst = make_worker_info([262144], [4096], 8, tp=4, rank=0)
    out = _sorted_by_src(_parse("RAGGED_PGTD", src, dst,
                                [TaskBuf(0, 8, False, [[0, 1, 2]], [[4, 5, 6]])])[0])
    assert out[:4] == [(0, 1048576, 512), (512, 1050624, 512), (1024, 1052672, 512),
                       (1536, 1054720, 512)]
    assert out[-1] == (7680, 1079296, 512)


# send_stub_test.cpp:499-705 (ParseBlockSendDGtP): P tp 4 -> D tp 16.
@pytest.mark.parametrize("d_rank", [0, 1, 2, 3, 7])
def test_ragged_p_lt_d_known_answer(d_rank):
    src = make_worker_info([4096 * 64], [4096], 8, tp=4, rank=d_rank // 4)
    dst = make_worker_info([1024 * 64], [1024], 8, tp=16, rank=d_rank)
    out = _parse("RAGGED_PLTD", src, dst, [TaskBuf(0, 8, False, [[0, 1, 2]], [[4, 5, 6]])],
                 valid=0xF, tp_size=4, tp_rank=d_rank // 4)
    g = d_rank % 4
    exp = []
    for t in range(8):
        exp.append((4096 * t + 512 * g, 262144 + 1024 * t, 512))
        exp.append((4096 * t + 2048 + 512 * g, 262144 + 1024 * t + 512, 512))
    assert _sorted_by_src(out[0]) == exp


# send_stub_test.cpp:707-1130 (ParseBlockSendPEqD): B = 16 KiB, T = 1 KiB, pool 16.
def _w16(**kw):
    return make_worker_info([16 * KB], [KB], 16, **kw)


def test_p_eq_d_chunk_sequence_shape1_ragged():
    B, T = 16 * KB, KB
    w = _w16()
    o = _parse("RAGGED_PEQD", w, w, [TaskBuf(0, 8, False, [[0, 1, 2]], [[4, 5, 6]])])
    assert o[0] == [(0, 65536, 8192)]
    o = _parse("RAGGED_PEQD", w, w, [TaskBuf(0, 17, False, [[0, 1, 2]], [[4, 5, 6]])])
    merged, stats = checkers.oracle_merge(np.array(o[0], dtype=np.uint64))
    assert [tuple(r) for r in merged.tolist()] == [(0, 65536, 17408)]
    assert stats == (17408, 17408, 17408, 1)
    o = _parse("RAGGED_PEQD", w, w, [TaskBuf(17, 16, True, [[3, 4, 5]], [[7, 8, 9]])])
    merged, _ = checkers.oracle_merge(np.array(o[0], dtype=np.uint64))
    assert [tuple(r) for r in merged.tolist()] == [(4 * B + T, 8 * B + T, 16 * T)]


def test_p_eq_d_chunk_sequence_shape2_flash():
    w = _w16()
    o = _parse("FLASH_PEQD", w, w, [TaskBuf(0, 8, False, [[0, 1, 2]], [[4, 5, 6]])])
    # K half-block 8 KiB, half-token 512 B; V = K + (B/2) * pool on both sides
    assert o[0] == [(0, 32768, 4096), (131072, 32768 + 131072, 4096)]


def test_p_eq_d_chunk_sequence_shape3_hybrid_pages():
    B = 16 * KB
    w = _w16(num_gdn_layers=0)
    # a partial first chunk that does not reach a page boundary sends nothing
    o = _parse("HYBRID_PEQD", w, w, [TaskBuf(0, 8, False, [[0, 1, 2]], [[4, 5, 6]])])
    assert o[0] == []
    # 17 tokens: one whole page, the 1-token tail is deferred
    o = _parse("HYBRID_PEQD", w, w, [TaskBuf(0, 17, False, [[0, 1, 2]], [[4, 5, 6]])])
    assert o[0] == [(0, 65536, 16384)]
    # last chunk with three GDN groups: attn pages 3,4,5 then GDN pages 6,7,8 merge into one run
    w3 = _w16(num_gdn_layers=3)
    o = _parse("HYBRID_PEQD", w3, w3,
               [TaskBuf(17, 16, True, [[6], [7], [8], [3, 4, 5]], [[10], [11], [12], [7, 8, 9]])])
    merged, _ = checkers.oracle_merge(np.array(o[0], dtype=np.uint64))
    assert [tuple(r) for r in merged.tolist()] == [(4 * B, 8 * B, 5 * B)]
    o = _parse("HYBRID_PEQD", w3, w3,
               [TaskBuf(1, 3, True, [[4], [5], [6], [3]], [[8], [9], [10], [7]])])
    merged, _ = checkers.oracle_merge(np.array(o[0], dtype=np.uint64))
    assert [tuple(r) for r in merged.tolist()] == [(3 * B, 7 * B, 4 * B)]


# send_stub_test.cpp:1565-1644 / :2280-2324 expect per-head records for the P==D
# FlashInfer hybrid shape, but the shipped parser copies whole pages
# (parse_block_qwen3_next_flashinfer.cpp:97-107); the code is followed.
def test_hybrid_flashinfer_p_eq_d_is_whole_pages():
    w = make_worker_info([16384], [1024], 16, num_kv_heads=4, num_gdn_layers=1)
    o = _parse("HYBRID_FI_PEQD", w, w,
               [TaskBuf(0, 20, True, [[6], [0, 1]], [[10], [4, 5]])])
    assert o[0] == [(0, 65536, 16384), (16384, 81920, 16384), (98304, 163840, 16384)]


# send_stub_test.cpp:1646-1755 (Qwen3NextFlashinferPGtD)
def test_hybrid_flashinfer_p_gt_d_known_answer():
    kw = dict(num_kv_heads=4, num_gdn_layers=1, conv_state_shape=[1, 3, 4],
              ssm_state_shape=[1, 1, 2, 2], gdn_conv_channel_dims=[2, 2])
    src = make_worker_info([2 * 1 * 64 * 2 * 16], [256], 256, tp=4, rank=0, **kw)
    dst = make_worker_info([2 * 2 * 64 * 2 * 16], [512], 256, tp=2, rank=0, **kw)
    valid = checkers.oracle().kvto_valid_ranks(4, 2, 4)
    assert valid == 0xF
    o = _parse("HYBRID_FI_PGTD", src, dst,
               [TaskBuf(0, 16, True, [[100], [0, 1]], [[200], [10, 11]])], valid=valid)[0]
    assert len(o) == 9
    assert sum(r[2] for r in o[:7]) == 16
    pB, dB = 4096, 8192
    assert o[7] == (0, 10 * dB, pB // 2)
    assert o[8] == (pB // 2, 10 * dB + dB // 2, pB // 2)
    # GDN P>D closed form (group_n 2, group_off 0): rows of 4 B split in two 2 B channels
    p, d = 100 * pB, 200 * dB
    exp = []
    for r in range(3):
        exp += [(p + 4 * r, d + 8 * r, 2), (p + 4 * r + 2, d + 8 * r + 4, 2)]
    exp.append((p + 12, d + 24, 4))
    assert o[:7] == exp


# parse_block_kda_test.cpp:78-361: SD conv state {8,2,6} x 1 B, recurrent {8,1,2,2} x 4 B,
# channel dims {2,2,2}, P tp 4 rank 1 -> D tp 2, pages of 32 B (P) and 64 B (D), block 1 -> 2
def test_kda_p_gt_d_sd_known_answer():
    kw = dict(num_gdn_layers=1, conv_state_shape=[8, 2, 6], ssm_state_shape=[8, 1, 2, 2],
              gdn_conv_channel_dims=[2, 2, 2], gdn_conv_elem_size=1, gdn_ssm_elem_size=4)
    src = make_worker_info([32], [32], 8, tp=4, rank=1, **kw)
    dst = make_worker_info([64], [64], 8, tp=2, rank=0, **kw)
    o = _parse("KDA_PGTD", src, dst, [TaskBuf(0, 1, True, [[1]], [[2]])])[0]
    assert o == [(32, 130, 2), (34, 134, 2), (36, 138, 2), (38, 142, 2), (40, 146, 2),
                 (42, 150, 2), (44, 168, 16)]
    # nothing is sent before the request's last chunk
    assert _parse("KDA_PGTD", src, dst, [TaskBuf(0, 1, False, [[1]], [[2]])])[0] == []


def test_kda_layout_closed_forms():
    # DS layout keeps each channel's history contiguous: one piece per q/k/v component
    kw = dict(num_gdn_layers=1, conv_state_shape=[8, 6, 2], ssm_state_shape=[8, 1, 2, 2],
              gdn_conv_channel_dims=[2, 2, 2], gdn_conv_elem_size=1, gdn_ssm_elem_size=4,
              kda_conv_dim_first=True)
    src = make_worker_info([32], [32], 8, tp=4, rank=1, **kw)
    dst = make_worker_info([64], [64], 8, tp=2, rank=0, **kw)
    o = _parse("KDA_PGTD", src, dst, [TaskBuf(0, 1, True, [[1]], [[2]])])[0]
    assert o == [(32, 128 + 4, 4), (36, 128 + 8 + 4, 4), (40, 128 + 16 + 4, 4), (44, 168, 16)]
    # P==D: whole pages, page stride override
    w = make_worker_info([32], [32], 16, kda_page_stride=48, **kw)
    o = _parse("KDA_PEQD", w, w, [TaskBuf(0, 1, True, [[3]], [[5]])])[0]
    assert o == [(144, 240, 48)]
    # P<D mirrors P>D: the receiver takes its slice of every component
    kw2 = dict(kw, conv_state_shape=[8, 12, 2], ssm_state_shape=[8, 2, 2, 2],
               gdn_conv_channel_dims=[4, 4, 4])
    srcw = make_worker_info([64], [64], 8, tp=2, rank=0, **kw2)
    dstn = make_worker_info([32], [32], 8, tp=4, rank=1, **kw2)
    o = _parse("KDA_PLTD", srcw, dstn, [TaskBuf(0, 1, True, [[2]], [[1]])], valid=0b11)[0]
    assert o == [(128 + 4, 32, 4), (128 + 8 + 4, 36, 4), (128 + 16 + 4, 40, 4), (128 + 24 + 16, 44, 16)]


# send_stub_test.cpp:1552-1559, :2739-2802 (ComputeValidRanksTest.*) and :1803-1807
@pytest.mark.parametrize("p,d,heads,mask", [
    (4, 2, 8, 0b1111), (8, 4, 8, 0xFF), (8, 4, -1, 0xFF), (8, 2, 2, 0b00010001),
    (8, 2, 4, 0b01010101), (8, 4, 2, 0b01010101), (2, 8, 4, 0b11), (4, 2, 2, 0b0101),
])
def test_valid_ranks_known_answers(p, d, heads, mask):
    assert checkers.oracle().kvto_valid_ranks(p, d, heads) == mask


# send_stub_test.cpp:1212-1277 (MergeIntervalTest); zero-length leftovers erased
@pytest.mark.parametrize("data,merged,stats", [
    ([], [], (2**64 - 1, 0, 0, 0)),
    ([(1, 1, 1)], [(1, 1, 1)], (1, 1, 1, 1)),
    ([(1, 1, 1), (3, 3, 2)], [(1, 1, 1), (3, 3, 2)], (1, 2, 3, 2)),
    ([(1, 1, 2), (3, 3, 1)], [(1, 1, 3)], (3, 3, 3, 1)),
    ([(1, 1, 2), (3, 3, 1), (4, 5, 2)], [(1, 1, 3), (4, 5, 2)], (2, 3, 5, 2)),
    ([(1, 1, 2), (1, 3, 1), (2, 4, 2)], [(1, 1, 2), (1, 3, 3)], (2, 3, 5, 2)),
])
def test_merge_known_answers(data, merged, stats):
    got, st = checkers.oracle_merge(np.array(data, dtype=np.uint64).reshape(-1, 3))
    assert [tuple(r) for r in got.tolist()] == merged
    assert st == stats


def test_merge_sorts_by_source_offset():
    got, _ = checkers.oracle_merge(np.array([(9, 0, 1), (2, 5, 3), (5, 8, 4)], dtype=np.uint64))
    assert [tuple(r) for r in got.tolist()] == [(2, 5, 7), (9, 0, 1)]


# send_stub_test.cpp:1141-1158: capacity src 1024 / dst 2048, source length scale 2
def test_bounds_known_answers():
    import ctypes as C
    lib = checkers.oracle()

    def ok(which, cap, scale, s, d, n):
        a = np.array([(s, d, n)], dtype=np.uint64)
        return lib.kvto_validate(a.ctypes.data, 1, cap, which, scale, None) == 0

    assert ok(0, 1024, 2, 0, 1024, 512) and ok(1, 2048, 1, 0, 1024, 512)
    assert not ok(0, 1024, 2, 1, 0, 512)
    assert not ok(1, 2048, 1, 0, 1537, 512)
    assert not ok(1, 2048, 1, 0, 0, 0)
    bad = C.c_uint64(99)
    a = np.array([(0, 0, 8), (0, 2041, 8)], dtype=np.uint64)
    assert lib.kvto_validate(a.ctypes.data, 2, 2048, 1, 1, C.byref(bad)) == 1 and bad.value == 1


def test_parse_rejects_out_of_pool_block_like_reference_bounds_check():
    w = make_worker_info([65536], [4096], 8)
    rc, _ = checkers.oracle_parse(PARSER["FLASH_PEQD"], w, w, 1, 1, 1 - 1,
                                  [TaskBuf(0, 16, True, [[8]], [[0]])])
    assert rc == 1


# Values produced by the compiled reference for configuration-shaped inputs.
def test_config_shaped_samples():
    w = make_worker_info([65536], [4096], 1024, num_kv_heads=8)
    o = _parse("FLASH_PEQD", w, w, [TaskBuf(0, 40, True, [[7, 3, 900]], [[0, 1, 2]])])[0]
    assert o == [(229376, 0, 32768), (98304, 32768, 32768), (29491200, 65536, 16384),
                 (33783808, 33554432, 32768), (33652736, 33587200, 32768),
                 (63045632, 33619968, 16384)]
    o = _parse("FLASHINFER_PEQD", w, w, [TaskBuf(0, 20, True, [[5, 2]], [[1, 0]])])[0]
    assert len(o) == 32
    for h in range(8):
        assert o[2 * h] == (327680 + 4096 * h, 65536 + 4096 * h, 4096)
        assert o[2 * h + 1] == (327680 + 32768 + 4096 * h, 65536 + 32768 + 4096 * h, 4096)
        assert o[16 + 2 * h] == (131072 + 4096 * h, 4096 * h, 1024)
        assert o[16 + 2 * h + 1] == (131072 + 32768 + 4096 * h, 32768 + 4096 * h, 1024)
    m = make_worker_info([36864, 8192], [576, 128], 64, num_kv_heads=1)
    o = _parse("DPSK_PEQD", m, m, [TaskBuf(10, 150, True, [[9, 3, 4]], [[7, 8, 1]])])
    assert o[0] == [(337536, 263808, 31104), (110592, 294912, 36864), (147456, 36864, 18432)]
    assert o[1] == [(75008, 58624, 6912), (24576, 65536, 8192), (32768, 8192, 4096)]
