"""Layer-message framing (TCP and staged-RDMA frames) and KVStore block-object
lists: the product's C-ABI functions against the format oracle
(oracle/kvt_wire_oracle.py) and against frames assembled by hand. CPU only."""
import ctypes as C
import os
import struct
import sys

import numpy as np
import pytest

import checkers
import kvt_amd
from kvt_amd import binding, workloads
from kvt_amd.binding import WIRE_RDMA_STAGED, WIRE_TCP

sys.path.insert(0, os.path.join(checkers.ROOT, "oracle"))
import kvt_wire_oracle as wo  # noqa: E402


def _lists(per_tensor):
    bl = kvt_amd.BlockLists()
    for t, runs in enumerate(per_tensor):
        bl.append(t, np.asarray(runs, dtype=np.uint64).reshape(-1, 3))
    return bl


def _frame(fmt, reqid, layer, per_tensor, blobs):
    bl = _lists(per_tensor)
    lay = binding.wire_layout_of(fmt, bl)
    buf = np.full(lay.total_bytes, 0xEE, dtype=np.uint8)
    lay2 = binding.wire_write_frame(fmt, buf.ctypes.data, len(buf), reqid, layer, bl)
    assert bytes(lay) == bytes(lay2)
    for t, blob in enumerate(blobs):
        assert lay.blob_bytes[t] == len(blob)
        buf[lay.blob_offset[t]:lay.blob_offset[t] + len(blob)] = np.frombuffer(blob, np.uint8)
    return buf, lay


# ---- the oracle itself, pinned by a frame spelled out byte by byte --------

HAND_TCP = bytes.fromhex(
    "6143564b"                      # magic 0x4B564361, little-endian
    "efcdab8967452301"              # reqid 0x0123456789abcdef
    "0500000000000000"              # layer_idx 5
    "0200000000000000"              # num_tensors 2
    "0200000000000000"              # tensor 0: 2 ranges
    "1000000000000000" "0001000000000000" "0300000000000000"    # (16, 256, 3)
    "4000000000000000" "0000000000000000" "0200000000000000"    # (64, 0, 2)
    "0500000000000000" "a1a2a3b1b2"                             # 5 blob bytes
    "0100000000000000"              # tensor 1: 1 range
    "0000000000000000" "0800000000000000" "0100000000000000"    # (0, 8, 1)
    "0100000000000000" "c1")
HAND_TCP_TENSORS = [([(16, 256, 3), (64, 0, 2)], bytes.fromhex("a1a2a3b1b2")),
                    ([(0, 8, 1)], bytes.fromhex("c1"))]

HAND_STAGED = bytes.fromhex(
    "6143564b" "0700000000000000"   # magic, reqid 7
    "3f00000000000000"              # actual_len = 12+8+8+8+24+3 = 63
    "0900000000000000"              # layer_idx 9
    "0100000000000000"              # 1 range
    "2000000000000000" "4000000000000000" "0300000000000000"    # (32, 64, 3)
    "d1d2d3")


def test_oracle_matches_hand_assembled_frames():
    assert wo.tcp_write(0x0123456789ABCDEF, 5, HAND_TCP_TENSORS) == HAND_TCP
    reqid, layer, ts = wo.tcp_read(HAND_TCP, 2)
    assert (reqid, layer) == (0x0123456789ABCDEF, 5)
    assert [(list(r), HAND_TCP[o:o + n]) for r, o, n in ts] == \
        [(list(r), b) for r, b in HAND_TCP_TENSORS]
    assert wo.staged_write(7, 9, [(32, 64, 3)], bytes.fromhex("d1d2d3")) == HAND_STAGED
    reqid, layer, ts = wo.staged_read(HAND_STAGED)
    assert (reqid, layer) == (7, 9) and ts == [([(32, 64, 3)], 60, 3)]


def test_product_writes_the_hand_assembled_frames():
    buf, lay = _frame(WIRE_TCP, 0x0123456789ABCDEF, 5, [r for r, _ in HAND_TCP_TENSORS],
                      [b for _, b in HAND_TCP_TENSORS])
    assert buf.tobytes() == HAND_TCP
    assert list(lay.blob_offset[:2]) == [92, 137] and lay.total_bytes == len(HAND_TCP)
    buf, lay = _frame(WIRE_RDMA_STAGED, 7, 9, [[(32, 64, 3)]], [bytes.fromhex("d1d2d3")])
    assert buf.tobytes() == HAND_STAGED


# ---- product vs oracle on seeded frames ----------------------------------

def _random_tensors(rng, n_tensors, max_runs):
    out = []
    for _ in range(n_tensors):
        n = int(rng.integers(0, max_runs + 1))
        runs = [(int(rng.integers(0, 1 << 40)), int(rng.integers(0, 1 << 40)),
                 int(rng.integers(1, 300))) for _ in range(n)]
        blob = rng.integers(0, 256, sum(r[2] for r in runs), dtype=np.uint8).tobytes()
        out.append((runs, blob))
    return out


@pytest.mark.parametrize("seed", range(12))
def test_tcp_frames_equal_oracle_and_parse_back(seed):
    rng = np.random.default_rng(seed)
    nt = int(rng.integers(1, 9))
    tensors = _random_tensors(rng, nt, 40)
    reqid, layer = int(rng.integers(0, 1 << 63)), int(rng.integers(0, 200))
    buf, lay = _frame(WIRE_TCP, reqid, layer, [r for r, _ in tensors], [b for _, b in tensors])
    assert buf.tobytes() == wo.tcp_write(reqid, layer, tensors)
    # receiver side, on the oracle's bytes
    frame = np.frombuffer(wo.tcp_write(reqid, layer, tensors), dtype=np.uint8)
    rc, r2, l2, lists, lay2 = binding.wire_parse_frame(WIRE_TCP, frame.ctypes.data, len(frame), nt)
    assert rc == 0 and (r2, l2) == (reqid, layer) and lay2.n_tensors == nt
    o_req, o_layer, o_ts = wo.tcp_read(frame.tobytes(), nt)
    for t, (runs, off, size) in enumerate(o_ts):
        assert np.array_equal(lists.tensor(t), np.asarray(runs, np.uint64).reshape(-1, 3))
        assert (lay2.blob_offset[t], lay2.blob_bytes[t]) == (off, size)
    assert lay2.total_bytes == len(frame)


@pytest.mark.parametrize("seed", range(6))
def test_staged_frames_equal_oracle_and_parse_back(seed):
    rng = np.random.default_rng(100 + seed)
    (runs, blob), = _random_tensors(rng, 1, 60)
    buf, lay = _frame(WIRE_RDMA_STAGED, seed, 3 + seed, [runs], [blob])
    exp = wo.staged_write(seed, 3 + seed, runs, blob)
    assert buf.tobytes() == exp
    # the receive buffer is usually larger than the frame: actual_len bounds it
    padded = np.frombuffer(exp + b"\x00" * 100, dtype=np.uint8)
    rc, r2, l2, lists, lay2 = binding.wire_parse_frame(WIRE_RDMA_STAGED, padded.ctypes.data,
                                                       len(padded))
    assert rc == 0 and (r2, l2) == (seed, 3 + seed)
    _, _, [(o_runs, off, size)] = wo.staged_read(padded.tobytes())
    assert np.array_equal(lists.tensor(0), np.asarray(o_runs, np.uint64).reshape(-1, 3))
    assert (lay2.blob_offset[0], lay2.blob_bytes[0], lay2.total_bytes) == (off, size, len(exp))


def test_every_truncation_of_a_tcp_frame_is_rejected_like_the_reference():
    tensors = HAND_TCP_TENSORS
    frame = wo.tcp_write(1, 2, tensors)
    for cut in range(len(frame)):
        part = np.frombuffer(frame[:cut] + b"\x00", dtype=np.uint8)  # keep a valid pointer
        rc, *_ = binding.wire_parse_frame(WIRE_TCP, part.ctypes.data, cut, 2)
        with pytest.raises(wo.FrameError):
            wo.tcp_read(frame[:cut], 2)
        assert rc == kvt_amd.ctypes_defs.ERR_INVALID, cut
    full = np.frombuffer(frame, dtype=np.uint8)
    assert binding.wire_parse_frame(WIRE_TCP, full.ctypes.data, len(full), 2)[0] == 0
    assert binding.wire_parse_frame(WIRE_TCP, full.ctypes.data, len(full), 3)[0] != 0
    assert "num_tensors" in kvt_amd.lib().kvt_last_error().decode()


def test_staged_frame_error_cases():
    frame = wo.staged_write(1, 2, [(0, 0, 4)], b"abcd")
    a = np.frombuffer(frame, dtype=np.uint8).copy()
    for cut in range(len(a)):
        assert binding.wire_parse_frame(WIRE_RDMA_STAGED, a.ctypes.data, cut)[0] != 0, cut
        with pytest.raises(wo.FrameError):
            wo.staged_read(frame[:cut])
    b = a.copy()
    b[0] ^= 1                                    # magic
    assert binding.wire_parse_frame(WIRE_RDMA_STAGED, b.ctypes.data, len(b))[0] != 0
    b = a.copy()
    b[12:20] = np.frombuffer(struct.pack("<Q", 40), np.uint8)   # actual_len < metadata end
    assert binding.wire_parse_frame(WIRE_RDMA_STAGED, b.ctypes.data, len(b))[0] != 0
    with pytest.raises(wo.FrameError):
        wo.staged_read(b.tobytes())
    # a huge range count must not overflow the size check
    b = a.copy()
    b[28:36] = 0xFF
    assert binding.wire_parse_frame(WIRE_RDMA_STAGED, b.ctypes.data, len(b))[0] != 0
    t = np.frombuffer(wo.tcp_write(1, 2, [([(0, 0, 4)], b"abcd")]), np.uint8).copy()
    t[28:36] = 0xFF
    assert binding.wire_parse_frame(WIRE_TCP, t.ctypes.data, len(t), 1)[0] != 0


def test_write_frame_argument_errors():
    bl = _lists([[(0, 0, 8)], [(0, 0, 8)]])
    small = np.zeros(16, np.uint8)
    lay = binding.WireLayout()
    L = kvt_amd.lib()
    assert L.kvt_wire_write_frame(WIRE_TCP, small.ctypes.data, 16, 0, 0, bl.h,
                                  C.byref(lay)) == kvt_amd.ctypes_defs.ERR_OUT_OF_RANGE
    assert L.kvt_wire_layout_of(WIRE_RDMA_STAGED, bl.h, C.byref(lay)) == kvt_amd.ctypes_defs.ERR_INVALID
    assert L.kvt_wire_layout_of(7, bl.h, C.byref(lay)) == kvt_amd.ctypes_defs.ERR_INVALID
    assert L.kvt_wire_layout_of(WIRE_TCP, kvt_amd.BlockLists().h,
                                C.byref(lay)) == kvt_amd.ctypes_defs.ERR_INVALID


def test_parse_rejects_blob_size_that_differs_from_the_ranges():
    frame = np.frombuffer(wo.tcp_write(1, 0, [([(0, 0, 4)], b"abcde")]), np.uint8)
    rc, *_ = binding.wire_parse_frame(WIRE_TCP, frame.ctypes.data, len(frame), 1)
    assert rc == kvt_amd.ctypes_defs.ERR_INVALID


def test_layout_of_a_full_size_batch_matches_register_data_arithmetic():
    """total = header + per tensor (8 + 24 n + 8 + blob)   (tcp_channel.cpp:433-446)"""
    from kvt_amd import pipeline
    w = workloads.deepseek_mla(n_layers=2, pool=1024, n_req=8, tokens=4096)
    lists, kind = pipeline.parse_batch(w.cache_shape, *w.worker_infos(), w.task_bufs())
    lay = binding.wire_layout_of(WIRE_TCP, lists)
    total = 12 + 16
    for t in range(w.n_tensors):
        runs = lists.tensor(t)
        total += 8 + 24 * len(runs) + 8 + int(runs[:, 2].sum())
    assert lay.total_bytes == total and lay.n_tensors == w.n_tensors


# ---- KVStore block objects ------------------------------------------------

def _info(block_sizes, nblk):
    w = kvt_amd.ctypes_defs.WorkerInfo()
    w.engine_tp_size, w.worker_tp_rank = 1, 0
    w.n_tensors = len(block_sizes)
    for i, b in enumerate(block_sizes):
        w.block_sizes[i] = b
        w.token_sizes[i] = b // 16
    w.layer_num_blocks = nblk
    w.num_layers = 1
    return w


def test_block_objects_of_the_two_plane_layout_equal_kvcache_colon_blkid():
    """file_backend.py:279 saves kvcache[:, blkid]; :232 loads it back."""
    rng = np.random.default_rng(5)
    nblk_s, nblk_d, bs, h, d = 13, 9, 16, 2, 8
    kv = rng.integers(0, 1 << 16, (2, nblk_s, bs, h, d), dtype=np.uint16)
    B = 2 * bs * h * d * 2
    src_ids = [7, 0, 12, 3]
    dst_ids = [1, 8, 2, 5]
    lists, ob = kvt_amd.block_object_lists(kvt_amd.ctypes_defs.SHAPE_FLASH, _info([B], nblk_s),
                                           _info([B], nblk_d), src_ids, dst_ids)
    assert ob == B
    runs = lists.tensor(0)
    blob = checkers.oracle_pack(kv.view(np.uint8).reshape(-1), runs)
    for i, b in enumerate(src_ids):
        assert blob[i * B:(i + 1) * B].tobytes() == kv[:, b].tobytes()
    # load: objects land in kvcache[:, dst]
    out = np.zeros((2, nblk_d, bs, h, d), dtype=np.uint16)
    checkers.oracle_unpack(out.view(np.uint8).reshape(-1), runs, blob)
    for s, t in zip(src_ids, dst_ids):
        assert np.array_equal(out[:, t], kv[:, s])
    untouched = [b for b in range(nblk_d) if b not in dst_ids]
    assert not out[:, untouched].any()


def test_block_objects_of_block_major_layouts_and_errors():
    B0, B1 = 4096, 512
    lists, ob = kvt_amd.block_object_lists(kvt_amd.ctypes_defs.SHAPE_FLASHINFER,
                                           _info([B0, B1], 10), _info([B0, B1], 20),
                                           [3, 9], [19, 0])
    assert ob == B0 + B1
    assert lists.tensor(0).tolist() == [[3 * B0, 19 * B0, B0], [9 * B0, 0, B0]]
    assert lists.tensor(1).tolist() == [[3 * B1, 19 * B1, B1], [9 * B1, 0, B1]]
    with pytest.raises(kvt_amd.KvtError):
        kvt_amd.block_object_lists(kvt_amd.ctypes_defs.SHAPE_FLASHINFER, _info([B0], 10),
                                   _info([B0], 20), [10], [0])
    with pytest.raises(kvt_amd.KvtError):
        kvt_amd.block_object_lists(kvt_amd.ctypes_defs.SHAPE_FLASHINFER, _info([B0], 10),
                                   _info([B0 * 2], 20), [1], [0])


def test_enlarge_block_ids_is_the_kvsbackend_formula():
    """res[i] = lst[i // n] * n + (i % n)   (kvsbackend.py:207-214)"""
    rng = np.random.default_rng(8)
    for n in (1, 2, 3, 8):
        lst = rng.integers(0, 1 << 20, 37).tolist()
        want = [lst[i // n] * n + (i % n) for i in range(len(lst) * n)]
        assert binding.enlarge_block_ids(lst, n).tolist() == want
    assert len(binding.enlarge_block_ids([], 4)) == 0
    with pytest.raises(kvt_amd.KvtError):
        binding.enlarge_block_ids([1 << 31], 4)          # does not fit 32 bits
    with pytest.raises(kvt_amd.KvtError):
        binding.enlarge_block_ids([1], 0)


def test_object_plan_tables_place_every_block_under_one_object():
    """Host-only plan: packed position of block i's part = i * object_stride (+ the offset
    inside the part), so that packing layer l with layer_stride = object_bytes builds
    [layer 0 part][layer 1 part]... per block."""
    B, nblk, L = 4096, 12, 3
    lists, ob = kvt_amd.block_object_lists(kvt_amd.ctypes_defs.SHAPE_FLASH, _info([B], nblk),
                                           _info([B], nblk), [5, 1, 9], [0, 2, 4])
    plan = kvt_amd.Plan(-1, lists, [B * nblk], [B * nblk], objects=(ob, L * ob))
    pack_t, unpack_t, cb, shapes = plan.host_tables()
    assert plan.layer_bytes == 2 * L * ob + ob
    got = sorted((int(c["packed"]), int(c["cache"]), int(c["len"])) for c in pack_t)
    half = B // 2
    want = []
    for i, b in enumerate([5, 1, 9]):
        want += [(i * L * ob, b * half, half), (i * L * ob + half, nblk * half + b * half, half)]
    assert got == sorted(want)
    with pytest.raises(kvt_amd.KvtError):
        kvt_amd.Plan(-1, lists, [B * nblk], [B * nblk], objects=(ob, ob - 1))
    with pytest.raises(kvt_amd.KvtError):
        kvt_amd.Plan(-1, lists, [B * nblk], [B * nblk], objects=(ob + 16, 8 * ob))
