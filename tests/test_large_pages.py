"""Pages of 4 GiB and more: the reference forms two products of ParseBlock in 32 bits
(parse_block_qwen3_next.cpp:376-413 the indexer's token term and length, :108-248 the
kernel-block index times the pack size). No input may exist on which product, oracle and the
compiled reference silently disagree: the second product cannot exceed 32 bits (shown here on
an 8 GiB page, all three implementations equal); the first wraps for indexer blocks of 4 GiB or
more, where the oracle follows the reference's wrapped numbers and the product refuses the
geometry when the parser is created. Host only."""
import pytest

import checkers
import kvt_amd
from kvt_amd.ctypes_defs import PARSER, TaskBuf, make_worker_info


def _hybrid_workers(p_tok, d_tok, ntpb, pack, indexer=None, blocks=4):
    kw = dict(num_kv_heads=8, num_gdn_layers=1, conv_state_shape=[1, 3, 4],
              ssm_state_shape=[1, 1, 2, 2], gdn_conv_channel_dims=[2, 2], attn_kernel_blk_ntpb=16,
              attn_pack_size=pack)
    if indexer:
        kw.update(indexer_blk_ntpb=indexer[0], hybrid_indexer_token_size=indexer[1])
    src = make_worker_info([p_tok * ntpb * pack], [p_tok], blocks, tp=4, rank=0, **kw)
    dst = make_worker_info([d_tok * ntpb * pack], [d_tok], blocks, tp=2, rank=0, **kw)
    return src, dst


def _all_three(parser, src, dst, task):
    """-> the ranges of oracle, product and (where it was built) compiled reference"""
    valid = checkers.oracle().kvto_valid_ranks(src.engine_tp_size, dst.engine_tp_size, 8)
    tps = bin(valid).count("1")
    rc, outs = checkers.oracle_parse(PARSER[parser], src, dst, valid, tps, 0, [task])
    assert rc == 0
    res = {"oracle": [tuple(int(x) for x in r) for r in outs[0]]}
    p = kvt_amd.Parser(PARSER[parser], src, dst, valid, tps, 0)
    lists = kvt_amd.BlockLists()
    assert p.parse(task.struct, lists) == 0
    res["product"] = [tuple(int(x) for x in r) for r in lists.tensor(0)]
    if checkers.ref() is not None:
        rc, outs = checkers.ref_parse(PARSER[parser], src, dst, valid, tps, 0, [task])
        assert rc == 0
        res["reference"] = [tuple(int(x) for x in r) for r in outs[0]]
    return res


def test_kernel_block_index_times_pack_size_on_an_8_gib_page():
    # 32 KiB (P) / 64 KiB (D) tokens, 4 layers packed per page, 65 536 tokens per layer and
    # page (the most the product accepts): P pages of 8 GiB, D pages of 16 GiB; the last tokens
    # of a page have the largest kernel-block index (4 095), times pack = 16 380
    ntpb = 1 << 16
    src, dst = _hybrid_workers(32768, 65536, ntpb, 4)
    assert int(src.block_sizes[0]) == 8 << 30
    task = TaskBuf(ntpb - 3, 6, False, [[7], [0, 1]], [[9], [2, 3]])
    res = _all_three("HYBRID_PGTD", src, dst, task)
    assert len(res["product"]) > 0
    assert max(r[0] for r in res["product"]) > (8 << 30)      # offsets beyond the first page
    for who, got in res.items():
        assert got == res["oracle"], who


def test_indexer_block_just_below_4_gib_is_identical_everywhere():
    tok, pn = 65536, 65535                                    # 4 GiB - 64 KiB per indexer block
    src, dst = _hybrid_workers(131072, 262144, 65536, 1, indexer=(pn, tok))   # 8 / 16 GiB pages
    task = TaskBuf(pn - 2, 4, False, [[7], [0, 1], [0, 1]], [[9], [2, 3], [2, 3]])
    res = _all_three("HYBRID_PGTD", src, dst, task)
    assert any(r[2] == 2 * tok for r in res["product"])      # the indexer ranges are there
    for who, got in res.items():
        assert got == res["oracle"], who


@pytest.mark.parametrize("parser", ["HYBRID_PGTD", "HYBRID_PLTD", "HYBRID_FI_PGTD", "HYBRID_FI_PLTD"])
def test_indexer_block_of_4_gib_is_refused_by_the_product(parser):
    tok, pn = 65536, 65536
    src, dst = _hybrid_workers(131072, 262144, 65536, 1, indexer=(pn, tok))   # 8 / 16 GiB pages
    if parser.endswith("PLTD"):
        src, dst = dst, src
    valid = checkers.oracle().kvto_valid_ranks(src.engine_tp_size, dst.engine_tp_size, 8)
    with pytest.raises(kvt_amd.KvtError) as e:
        kvt_amd.Parser(PARSER[parser], src, dst, valid, bin(valid).count("1"), 0)
    assert e.value.code == 2 and "4 GiB" in str(e.value)


def test_what_the_refusal_avoids_the_reference_wraps():
    """The same 4 GiB indexer block through the oracle (and the compiled reference, where
    built): a whole-block range comes out with length 0 or is refused by the range check,
    because 65 536 tokens x 65 536 bytes is 0 in 32 bits -- the numbers the product declines
    to reproduce."""
    tok, pn = 65536, 65536
    src, dst = _hybrid_workers(131072, 262144, 65536, 1, indexer=(pn, tok))   # 8 / 16 GiB pages
    task = TaskBuf(0, pn, False, [[7], [0], [0]], [[9], [2], [2]])
    valid = checkers.oracle().kvto_valid_ranks(4, 2, 8)
    rc_o, outs_o = checkers.oracle_parse(PARSER["HYBRID_PGTD"], src, dst, valid, 4, 0, [task])
    assert rc_o == 1                       # length 0: "range validation failed" (std::out_of_range)
    if checkers.ref() is not None:
        rc_r, _ = checkers.ref_parse(PARSER["HYBRID_PGTD"], src, dst, valid, 4, 0, [task])
        assert rc_r == rc_o
