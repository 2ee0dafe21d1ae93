"""CPU restatement of the reference's per-layer wire frames (test infrastructure
only: nothing but tests/ may import this file; the product's framing lives in
llumnix-kv_amd/csrc/kvt_wire.cpp).

Writer and reader are restated separately, each from its own reference function,
so that a write -> read round trip cross-checks the two restatements:

* ``tcp_write``   TCPChannel::send_data          kvtransfer/src/tcp_channel.cpp:503-536
  (buffer size: register_data, :433-446)
* ``tcp_read``    TCPServer::CtxCallback::handle_kv_cache_data
                                                 kvtransfer/src/tcp_channel.cpp:149-225
* ``staged_write`` RDMAStagedChannel::send_data  kvtransfer/src/rdma_staged_channel.cpp:246-300
* ``staged_read``  RDMAStagedServer layer handler kvtransfer/src/rdma_staged_server.cpp:379-420
* header: ser_rpc_header / RPC_HEADER = u32 magic + u64 reqid; KV_CACHE_DATA_MAGIC
                                                 kvtransfer/include/copy_utils.h:32

What pins it: the reference holds no recorded frames, so tests/test_wire.py pins
this file with frames assembled by hand, byte by byte, plus the write/read
cross-check. ``size_t`` is 8 bytes little-endian on every platform the reference
builds for.
"""
import struct

MAGIC = 0x4B564361
RPC_HEADER = 12


class FrameError(ValueError):
    pass


def _ranges_bytes(runs):
    return b"".join(struct.pack("<QQQ", int(s), int(d), int(n)) for s, d, n in runs)


def tcp_write(reqid, layer_idx, tensors):
    """tensors: list of (runs [(src,dst,len)...], blob bytes)."""
    out = [struct.pack("<IQ", MAGIC, reqid), struct.pack("<QQ", layer_idx, len(tensors))]
    for runs, blob in tensors:
        out.append(struct.pack("<Q", len(runs)))
        out.append(_ranges_bytes(runs))
        out.append(struct.pack("<Q", len(blob)))
        out.append(bytes(blob))
    return b"".join(out)


def tcp_read(buf, expect_tensors):
    """-> (reqid, layer_idx, [(runs, blob_offset, blob_bytes)...]); FrameError where the
    reference's handler logs an error and drops the message."""
    n = len(buf)
    if n < RPC_HEADER + 16:
        raise FrameError("message too short")
    magic, reqid = struct.unpack_from("<IQ", buf, 0)
    if magic != MAGIC:
        raise FrameError("bad magic")
    layer_idx, num_tensors = struct.unpack_from("<QQ", buf, RPC_HEADER)
    if num_tensors != expect_tensors:
        raise FrameError("num_tensors mismatch")
    pos = RPC_HEADER + 16
    res = []
    for _ in range(num_tensors):
        if pos + 8 > n:
            raise FrameError("truncated at metadata_size")
        (cnt,) = struct.unpack_from("<Q", buf, pos)
        pos += 8
        if pos + cnt * 24 + 8 > n:
            raise FrameError("incomplete metadata")
        runs = [struct.unpack_from("<QQQ", buf, pos + 24 * i) for i in range(cnt)]
        pos += cnt * 24
        (size,) = struct.unpack_from("<Q", buf, pos)
        pos += 8
        if pos + size > n:
            raise FrameError("truncated tensor data")
        res.append((runs, pos, size))
        pos += size
    return reqid, layer_idx, res


def staged_write(reqid, layer_idx, runs, blob):
    meta = struct.pack("<Q", len(runs)) + _ranges_bytes(runs)
    total = RPC_HEADER + 8 + 8 + len(meta) + len(blob)
    return (struct.pack("<IQ", MAGIC, reqid) + struct.pack("<QQ", total, layer_idx) + meta
            + bytes(blob))


def staged_read(buf):
    n = len(buf)
    if n < RPC_HEADER + 24:
        raise FrameError("message too short")
    magic, reqid = struct.unpack_from("<IQ", buf, 0)
    if magic != MAGIC:
        raise FrameError("bad magic")
    actual_len, layer_idx, cnt = struct.unpack_from("<QQQ", buf, RPC_HEADER)
    if actual_len > n:
        raise FrameError("stated length exceeds the message")
    expected_len = RPC_HEADER + 24 + cnt * 24
    if actual_len < expected_len:
        raise FrameError("incomplete metadata")
    runs = [struct.unpack_from("<QQQ", buf, RPC_HEADER + 24 + 24 * i) for i in range(cnt)]
    return reqid, layer_idx, [(runs, expected_len, actual_len - expected_len)]
