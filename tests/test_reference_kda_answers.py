"""Every expectation of the reference's KDA / Kimi-K3 parser tests
(kvtransfer/tests/parse_block_kda_test.cpp:78-361), checked against the CPU oracle and
against the product parser through the C ABI. The fixture of those tests fills the layout
fields on the SOURCE WorkerInfo only and leaves attn_kernel_blk_ntpb at 0 unless a test
sets it; the same is done here."""
import checkers
import kvt_amd
from kvt_amd.ctypes_defs import PARSER, TaskBuf, make_worker_info


def _fixture(p_tp, p_rank, d_tp, d_rank, pB, dB, layout=None, kimi=None):
    """KdaParseFixture (parse_block_kda_test.cpp:8-65) + configure_kimi_mla (:199-218).
    layout = (conv_shape, recurrent_shape, channel_dims, dim_first); kimi = (kernel_ntpb,
    manager_ntpb)."""
    s_kw = dict(num_gdn_layers=1, attn_kernel_blk_ntpb=0)
    d_kw = dict(num_gdn_layers=3, attn_kernel_blk_ntpb=0)
    if layout is not None:
        conv, rec, chans, dim_first = layout
        s_kw.update(conv_state_shape=conv, ssm_state_shape=rec, gdn_conv_channel_dims=chans,
                    gdn_conv_elem_size=1, gdn_ssm_elem_size=4, kda_conv_dim_first=dim_first)
    pT = dT = 1
    if kimi is not None:
        kernel_ntpb, manager_ntpb = kimi
        for kw, B in ((s_kw, pB), (d_kw, dB)):
            kw.update(attn_kernel_blk_ntpb=kernel_ntpb, hybrid_attn_token_size=2, kda_page_stride=B)
        pT, dT = pB // manager_ntpb, dB // manager_ntpb
    src = make_worker_info([pB], [pT], 8, tp=p_tp, rank=p_rank, **s_kw)
    dst = make_worker_info([dB], [dT], 8, tp=d_tp, rank=d_rank, **d_kw)
    return src, dst


def _run(parser, src, dst, task, valid, tp_size, tp_rank):
    # the Kimi-K3 cases name the parser the dispatch must pick for these two workers (the rank
    # values are literals of the reference tests, not derived from the workers)
    checkers.assert_dispatch(parser, src, dst)
    rc, outs = checkers.oracle_parse(PARSER[parser], src, dst, valid, tp_size, tp_rank, [task])
    assert rc == 0 and len(outs) == 1
    oracle = [tuple(int(x) for x in r) for r in outs[0]]
    p = kvt_amd.Parser(PARSER[parser], src, dst, valid, tp_size, tp_rank)
    lists = kvt_amd.BlockLists()
    assert p.parse(task.struct, lists) == 0
    product = [tuple(int(x) for x in r) for r in lists.tensor(0)] if lists.num_tensors() else []
    assert product == oracle
    return oracle


def _task(src_groups=((1,),), dst_groups=((2,),), seen=0, new=1, last=True):
    return TaskBuf(seen, new, last, [list(g) for g in src_groups], [list(g) for g in dst_groups])


SD_NARROW = ([8, 2, 6], [8, 1, 2, 2], [2, 2, 2], False)
DS_NARROW = ([8, 6, 2], [8, 1, 2, 2], [2, 2, 2], True)
SD_WIDE = ([8, 2, 12], [8, 2, 2, 2], [4, 4, 4], False)
DS_WIDE = ([8, 12, 2], [8, 2, 2, 2], [4, 4, 4], True)


def test_kda_p_eq_d_copies_the_full_padded_page():                       # :78-92
    src, dst = _fixture(2, 1, 2, 1, 64, 64)
    assert _run("KDA_PEQD", src, dst, _task(), 0, 2, 1) == [(64, 128, 64)]


def test_kda_p_gt_d_merges_sd_qkv_rows_and_recurrent_heads():            # :94-118
    src, dst = _fixture(4, 1, 2, 0, 32, 64, SD_NARROW)
    assert _run("KDA_PGTD", src, dst, _task(), 0, 0, 0) == [
        (32, 130, 2), (34, 134, 2), (36, 138, 2), (38, 142, 2), (40, 146, 2), (42, 150, 2),
        (44, 168, 16)]


def test_kda_p_gt_d_merges_ds_qkv_components_and_recurrent_heads():      # :120-141
    src, dst = _fixture(4, 1, 2, 0, 32, 64, DS_NARROW)
    assert _run("KDA_PGTD", src, dst, _task(), 0, 0, 0) == [
        (32, 132, 4), (36, 140, 4), (40, 148, 4), (44, 168, 16)]


def test_kda_p_lt_d_splits_sd_qkv_rows_and_recurrent_heads():            # :143-167
    src, dst = _fixture(2, 0, 4, 1, 64, 32, SD_WIDE)
    assert _run("KDA_PLTD", src, dst, _task(), 0, 0, 0) == [
        (66, 64, 2), (70, 66, 2), (74, 68, 2), (78, 70, 2), (82, 72, 2), (86, 74, 2),
        (104, 76, 16)]


def test_kda_p_lt_d_splits_ds_qkv_components_and_recurrent_heads():      # :169-190
    src, dst = _fixture(2, 0, 4, 1, 64, 32, DS_WIDE)
    assert _run("KDA_PLTD", src, dst, _task(), 0, 0, 0) == [
        (68, 64, 4), (76, 68, 4), (84, 72, 4), (104, 76, 16)]


def test_kda_does_not_send_mutable_state_before_the_request_finishes():  # :192-205
    src, dst = _fixture(2, 0, 2, 0, 64, 64)
    assert _run("KDA_PEQD", src, dst, _task(last=False), 0, 2, 0) == []


TWO_GROUPS = dict(src_groups=((1,), (3,)), dst_groups=((2,), (4,)))


def test_kimi_p_eq_d_copies_mla_prefix_and_kda_page():                   # :220-240
    src, dst = _fixture(2, 1, 2, 1, 64, 64, kimi=(4, 4))
    assert _run("KIMI_K3_PEQD", src, dst, _task(**TWO_GROUPS), 0b11, 2, 1) == [
        (3 * 64, 4 * 64, 8), (1 * 64, 2 * 64, 64)]


def test_kimi_p_eq_d_uses_the_block_manager_granularity():               # :242-276
    src, dst = _fixture(2, 1, 2, 1, 64, 64, kimi=(2, 4))
    groups = dict(src_groups=((1,), (3, 5)), dst_groups=((2,), (4, 6)))
    # completing one attention kernel block sends nothing of the four-token manager block
    assert _run("KIMI_K3_PEQD", src, dst, _task(seen=0, new=2, last=False, **groups),
                0b11, 2, 1) == []
    assert _run("KIMI_K3_PEQD", src, dst, _task(seen=2, new=1, last=True, **groups),
                0b11, 2, 1) == [(3 * 64, 4 * 64, 8), (5 * 64, 6 * 64, 8), (1 * 64, 2 * 64, 64)]


def test_kimi_p_gt_d_merges_kda_and_copies_mla_from_the_representative():  # :278-304
    src, dst = _fixture(4, 0, 2, 0, 32, 64, SD_NARROW, kimi=(4, 4))
    o = _run("KIMI_K3_PGTD", src, dst, _task(**TWO_GROUPS), 0b0101, 2, 0)
    assert len(o) == 9
    assert o[0] == (3 * 32, 4 * 64, 8)
    assert o[1] == (3 * 32, 4 * 64 + 2, 6)        # the remaining 3 D tokens, from block 0
    assert o[-1] == (32 + 12, 2 * 64 + 24, 16)


def test_kimi_p_gt_d_skips_replicated_mla_on_the_other_rank():           # :306-330
    src, dst = _fixture(4, 1, 2, 0, 32, 64, SD_NARROW, kimi=(4, 4))
    o = _run("KIMI_K3_PGTD", src, dst, _task(**TWO_GROUPS), 0b0101, 2, 1)
    assert len(o) == 7 and all(r[0] != 3 * 32 for r in o)


def test_kimi_p_lt_d_splits_kda_and_fans_out_mla():                      # :332-358
    src, dst = _fixture(2, 0, 4, 1, 64, 32, SD_WIDE, kimi=(4, 4))
    o = _run("KIMI_K3_PLTD", src, dst, _task(**TWO_GROUPS), 0b11, 2, 0)
    assert len(o) == 9
    assert o[0] == (3 * 64, 4 * 32, 8)
    assert o[1] == (3 * 64, 4 * 32 + 2, 6)
    assert o[-1] == (64 + 40, 2 * 32 + 12, 16)
