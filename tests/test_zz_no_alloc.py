"""kvt_copy_handle_data_kernel_direct_static: the variant of
kvt_copy_handle_data_kernel_direct whose device-side range metadata lives in an array that is
part of the library's code object, for callers that cannot allocate (graph capture, serving
loops, harnesses that forbid hipMalloc). Called through the C ABI; every result must equal,
byte for byte, what the existing entry point produces on the same input, on two calls in a
row of which the second is smaller, in both directions. Needs a real MI355X."""
import numpy as np
import pytest

import checkers
import kvt_amd

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

CAP = 1 << 22


def _ranges(seed, n, explicit):
    """n ranges of 1..6000 bytes at ascending cache offsets with gaps; the contiguous side as a
    running sum, or shuffled with gaps (explicit offsets)."""
    rng = np.random.default_rng(seed)
    lens = rng.integers(1, 6000, n).astype(np.uint64)
    gpu_off = (np.cumsum(lens + rng.integers(0, 3000, n).astype(np.uint64)) - lens).astype(np.uint64)
    assert int(gpu_off[-1] + lens[-1]) <= CAP
    if explicit:
        host_off, cur = np.zeros(n, dtype=np.uint64), 0
        for i in rng.permutation(n):
            host_off[i] = cur
            cur += int(lens[i]) + int(rng.integers(0, 64))
        size = cur
    else:
        host_off, size = np.zeros(n, dtype=np.uint64), int(lens.sum())
    return np.ascontiguousarray(np.stack([host_off, gpu_off, lens], axis=1)), size


def _both_entry_points(lib, st, blocks, size, layer, explicit):
    """-> (gathered bytes, scattered cache) of the existing entry point and of the static one"""
    n = len(blocks)
    dev = [torch.zeros(n, dtype=torch.int64, device="cuda") for _ in range(3)]
    host_meta = torch.zeros(3 * n, dtype=torch.int64).pin_memory()
    out = []
    for static in (False, True):
        pinned = torch.full((size,), 0x11, dtype=torch.uint8).pin_memory()
        dst = torch.full((CAP,), 0x33, dtype=torch.uint8, device="cuda")
        for buf, gpu, direction in ((pinned, layer, 1), (pinned, dst, 0)):
            if static:
                rc = lib.kvt_copy_handle_data_kernel_direct_static(
                    buf.data_ptr(), gpu.data_ptr(), blocks.ctypes.data, n, size, direction, 0,
                    st.cuda_stream, host_meta.data_ptr(), 1 if explicit else 0)
            else:
                rc = lib.kvt_copy_handle_data_kernel_direct(
                    buf.data_ptr(), gpu.data_ptr(), blocks.ctypes.data, n, size, direction, 0,
                    st.cuda_stream, dev[0].data_ptr(), dev[1].data_ptr(), dev[2].data_ptr(),
                    host_meta.data_ptr(), 1 if explicit else 0)
            assert rc == 0, lib.kvt_last_error()
            st.synchronize()      # host_meta is reused by the next call
        out.append((pinned.numpy().copy(), dst.cpu().numpy()))
    return out


@pytest.mark.parametrize("explicit", [False, True])
def test_static_metadata_entry_point_equals_the_existing_one(explicit):
    lib = kvt_amd.lib()
    assert lib.kvt_initialize_copy_method_profile(0) == 0, lib.kvt_last_error()
    st = checkers.side_stream()
    g = torch.Generator(device="cuda")
    g.manual_seed(91)
    layer = torch.randint(0, 256, (CAP,), generator=g, device="cuda", dtype=torch.uint8)
    layer_h = layer.cpu().numpy()
    # two calls in a row on the same GPU: the second is smaller and finds the first one's
    # metadata still in the array
    for seed, n in ((1, 700), (2, 90)):
        blocks, size = _ranges(seed, n, explicit)
        (ref_buf, ref_dst), (got_buf, got_dst) = _both_entry_points(lib, st, blocks, size, layer,
                                                                    explicit)
        assert np.array_equal(got_buf, ref_buf), (seed, "gather differs")
        assert np.array_equal(got_dst, ref_dst), (seed, "scatter differs")
        # and both are what the ranges say
        cur = 0
        for host_off, gpu_off, m in blocks.tolist():
            a = host_off if explicit else cur
            assert np.array_equal(got_buf[a:a + m], layer_h[gpu_off:gpu_off + m])
            assert np.array_equal(got_dst[gpu_off:gpu_off + m], layer_h[gpu_off:gpu_off + m])
            cur += m
        touched = np.zeros(CAP, dtype=bool)
        for _, gpu_off, m in blocks.tolist():
            touched[gpu_off:gpu_off + m] = True
        assert (got_dst[~touched] == 0x33).all()


def test_calls_on_two_streams_do_not_overwrite_each_others_metadata():
    """The reference's callers are several copy threads with a stream each
    (kvtransfer/src/copy_utils.cpp:59-154). Two streams issue different lists back to back
    while the first stream is held back by a sleeping kernel, so that without ordering the
    second call's metadata would replace the first one's before its kernel has run. Every call
    must still move its own ranges: results equal the existing entry point's."""
    lib = kvt_amd.lib()
    s1, s2 = checkers.side_stream(), checkers.side_stream()
    g = torch.Generator(device="cuda")
    g.manual_seed(92)
    layer = torch.randint(0, 256, (CAP,), generator=g, device="cuda", dtype=torch.uint8)
    cases = [_ranges(5, 700, False), _ranges(6, 400, True), _ranges(7, 90, False)]
    ref = [_both_entry_points(lib, s1, b, size, layer, ex)[0] for (b, size), ex in
           zip(cases, (False, True, False))]
    metas = [torch.zeros(3 * len(b), dtype=torch.int64).pin_memory() for b, _ in cases]
    bufs = [torch.full((size,), 0x11, dtype=torch.uint8).pin_memory() for _, size in cases]
    dsts = [torch.full((CAP,), 0x33, dtype=torch.uint8, device="cuda") for _ in cases]

    def call(i, stream, direction, gpu):
        b, size = cases[i]
        rc = lib.kvt_copy_handle_data_kernel_direct_static(
            bufs[i].data_ptr(), gpu.data_ptr(), b.ctypes.data, len(b), size, direction, 0,
            stream.cuda_stream, metas[i].data_ptr(), 1 if i == 1 else 0)
        assert rc == 0, lib.kvt_last_error()

    with torch.cuda.stream(s1):
        torch.cuda._sleep(100_000_000)              # stream 1 falls behind
    call(0, s1, 1, layer)                           # gathers, alternating streams, no waits
    call(1, s2, 1, layer)
    call(2, s1, 1, layer)
    s1.synchronize()
    s2.synchronize()
    with torch.cuda.stream(s2):
        torch.cuda._sleep(100_000_000)
    call(0, s2, 0, dsts[0])                         # scatters of what was gathered
    call(1, s1, 0, dsts[1])
    call(2, s2, 0, dsts[2])
    s1.synchronize()
    s2.synchronize()
    for i in range(3):
        assert np.array_equal(bufs[i].numpy(), ref[i][0]), (i, "gather differs")
        assert np.array_equal(dsts[i].cpu().numpy(), ref[i][1]), (i, "scatter differs")


def test_static_metadata_entry_point_refuses_what_it_cannot_hold():
    lib = kvt_amd.lib()
    st = checkers.side_stream()
    n = 8193
    blocks = np.ascontiguousarray(np.stack([np.zeros(n, np.uint64), np.arange(n, dtype=np.uint64) * 16,
                                            np.full(n, 16, np.uint64)], axis=1))
    layer = torch.zeros(n * 16, dtype=torch.uint8, device="cuda")
    pinned = torch.zeros(n * 16, dtype=torch.uint8).pin_memory()
    host_meta = torch.zeros(3 * n, dtype=torch.int64).pin_memory()
    rc = lib.kvt_copy_handle_data_kernel_direct_static(
        pinned.data_ptr(), layer.data_ptr(), blocks.ctypes.data, n, n * 16, 1, 0, st.cuda_stream,
        host_meta.data_ptr(), 0)
    assert rc == 3 and b"8192" in lib.kvt_last_error()
    # exactly the maximum is accepted
    n = 8192
    rc = lib.kvt_copy_handle_data_kernel_direct_static(
        pinned.data_ptr(), layer.data_ptr(), blocks.ctypes.data, n, n * 16, 1, 0, st.cuda_stream,
        host_meta.data_ptr(), 0)
    assert rc == 0, lib.kvt_last_error()
    st.synchronize()
