"""Closed forms of the cache geometry (kvt_amd.geometry) against the numbers
the benchmark configurations fix, and their error cases. CPU only."""
import pytest

from kvt_amd import geometry as G
from kvt_amd import workloads as W


def test_flash_attention_llama8b():
    # bf16 [2, nblk, 16, 8, 128]: 4096 B per token, 64 KiB per block
    tok = G.token_bytes([(2, 1024, 16, 8, 128)], [2])
    assert tok == [4096]
    blk = G.block_bytes(tok, 16)
    assert blk == [65536]
    nbytes = 2 * 1024 * 16 * 8 * 128 * 2
    assert G.layer_num_blocks([nbytes] * 32, blk[0]) == 1024
    w = W.llama8b_single()
    assert w.src_info["token_sizes"] == tok and w.src_info["block_sizes"] == blk
    assert w.src_info["layer_num_blocks"] == 1024


def test_flashinfer_logical_shape_gives_the_same_sizes():
    assert G.token_bytes([(8192, 2, 16, 8, 128)], [2]) == [4096]
    w = W.llama70b_flashinfer()
    assert w.src_info["token_sizes"] == [4096] and w.src_info["block_sizes"] == [65536]


def test_mla_and_sparse_mla_with_indexer():
    assert G.token_bytes([(4608, 64, 576)], [1]) == [576]
    tok = G.token_bytes([(4608, 64, 576), (4608, 64, 128)], [1, 1])
    assert tok == [576, 128]
    assert G.block_bytes(tok, 64) == [36864, 8192]
    w = W.deepseek_mla()
    assert w.src_info["token_sizes"] == tok and w.src_info["block_sizes"] == [36864, 8192]


def test_hybrid_pages_bundle_packed_layers():
    tok = G.token_bytes([(36864, 2, 16, 2, 256)], [2])
    assert tok == [2048]
    assert G.block_bytes(tok, 16, attn_pack_size=1, hybrid=True) == [32768]
    assert G.block_bytes(tok, 16, attn_pack_size=4, hybrid=True) == [131072]
    assert G.block_bytes(tok, 16, attn_pack_size=4, hybrid=False) == [32768]
    assert W.qwen3next_attn().src_info["block_sizes"] == [32768]


def test_errors():
    with pytest.raises(ValueError):
        G.token_bytes([(1, 2, 3, 4)], [2])
    with pytest.raises(ValueError):
        G.token_bytes([(2, 4, 16, 8, 128), (4, 64, 128)], [2, 1])
    with pytest.raises(ValueError):
        G.layer_num_blocks([1000], 0)
    with pytest.raises(ValueError):
        G.layer_num_blocks([65536, 65536 * 2], 65536)
    with pytest.raises(ValueError):
        G.layer_num_blocks([65536 + 1], 65536)
