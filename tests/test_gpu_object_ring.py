"""The pinned object ring on the GPU: what FileBackend does with blocks and their hashes
(blade_kvt/hybrid_connector/file_backend.py:215-285: save kvcache[:, blkid] of every layer
under the block's hash unless it is stored already, load it back into whatever block the
request was given) through one pack launch per batch, DMA copies into / out of ring entries,
and one unpack launch. Checked against torch's own kvcache[:, b] slices. Needs a real MI355X."""
import numpy as np
import pytest

import checkers
import kvt_amd

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

N_LAYERS, NBLK, BS, H, D = 4, 24, 16, 2, 64
B = 2 * BS * H * D * 2                     # one block of one layer (K and V), bytes
ENTRY = N_LAYERS * B                       # one block of all layers


def key(i):
    return int(i).to_bytes(8, "little") + b"blockkey"


def _caches(seed):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    kv = [torch.randn((2, NBLK, BS, H, D), generator=g, device="cuda").to(torch.bfloat16)
          for _ in range(N_LAYERS)]
    torch.cuda.synchronize()
    return kv


def _cache_handle(kv):
    return kvt_amd.Cache(0, [[k.view(torch.uint8).reshape(-1)] for k in kv], [B * NBLK])


def _plan(src_ids, dst_ids):
    info = kvt_amd.ctypes_defs.make_worker_info(block_sizes=[B], token_sizes=[B // BS],
                                                layer_num_blocks=NBLK, num_layers=N_LAYERS)
    lists, ob = kvt_amd.block_object_lists(kvt_amd.ctypes_defs.SHAPE_FLASH, info, info,
                                           np.asarray(src_ids), np.asarray(dst_ids))
    assert ob == B
    return kvt_amd.Plan(0, lists, [B * NBLK], [B * NBLK], objects=(ob, ENTRY))


def _object_of(kv, b):
    return torch.stack([kv[l][:, int(b)] for l in range(N_LAYERS)]).contiguous() \
        .view(torch.uint8).reshape(-1).cpu().numpy()


def _save(ring, kv, cache, blocks, keys, stream, pad=0):
    """One save step of a batch: ask the ring which blocks it lacks, pack those, hand them over."""
    entries, new = ring.reserve(keys)
    todo = [b for b, n in zip(blocks, new) if n]
    if todo:
        stride = ENTRY + pad
        objs = torch.zeros(len(todo) * stride, dtype=torch.uint8, device="cuda")
        torch.cuda.synchronize()            # the fill runs on torch's stream, the pack on `stream`
        plan = _plan(todo, todo)
        if pad == 0:
            plan.pack(cache, 0, N_LAYERS, objs, B, stream.cuda_stream)
        else:                               # objects spaced wider apart than an entry: one by one
            for i, b in enumerate(todo):
                p1 = _plan([b], [b])
                p1.pack(cache, 0, N_LAYERS, objs[i * stride:], B, stream.cuda_stream)
        ring.save(entries[new], objs.data_ptr(), stride, stream.cuda_stream)
        stream.synchronize()
    return entries, new


def test_save_by_hash_skips_stored_blocks_and_load_restores_them_elsewhere():
    kv = _caches(5)
    cache = _cache_handle(kv)
    ring = kvt_amd.ObjectRing(0, ENTRY, 8, 16)
    s = checkers.side_stream()
    blocks1, keys1 = [7, 3, 20, 11, 0], [key(i) for i in range(5)]
    e1, new1 = _save(ring, kv, cache, blocks1, keys1, s)
    assert e1.tolist() == [0, 1, 2, 3, 4] and new1.all()
    for b, idx in zip(blocks1, e1):
        ring.wait(idx)
        assert np.array_equal(ring.entry(idx), _object_of(kv, b)), b

    # second batch: two blocks are stored already (same hashes), four are new and wrap around
    blocks2, keys2 = [11, 0, 5, 6, 23, 9], [key(i) for i in (3, 4, 5, 6, 7, 8)]
    e2, new2 = _save(ring, kv, cache, blocks2, keys2, s)
    assert new2.tolist() == [False, False, True, True, True, True]
    assert e2.tolist() == [3, 4, 5, 6, 7, 0]              # key 0's entry was the oldest
    for b, idx in zip(blocks2, e2):
        ring.wait(idx)
        assert np.array_equal(ring.entry(idx), _object_of(kv, b)), b

    # a request that hits four stored blocks and two that are not there (one evicted, one unknown)
    want_keys = [key(8), key(3), key(0), key(1), key(6), key(99)]
    src_block_of = {8: 9, 3: 11, 1: 3, 6: 6}
    e, found = ring.lookup(want_keys)
    assert found.tolist() == [True, True, False, True, True, False]
    hit = e[found]
    assert hit.tolist() == [0, 3, 1, 6]
    new_cache = [torch.zeros_like(k) for k in kv]
    torch.cuda.synchronize()
    dst_blocks = [2, 19, 8, 14]
    objs = torch.empty(len(hit) * ENTRY, dtype=torch.uint8, device="cuda")
    hit_keys = [k for k, f in zip(want_keys, found) if f]
    with pytest.raises(kvt_amd.KvtError) as ex:           # the entries do not hold these keys
        ring.load(hit, objs.data_ptr(), ENTRY, s.cuda_stream, keys=hit_keys[::-1])
    assert ex.value.code == 1 and "given to another block" in str(ex.value)
    ring.load(hit, objs.data_ptr(), ENTRY, s.cuda_stream, keys=hit_keys)
    _plan(dst_blocks, dst_blocks).unpack(_cache_handle(new_cache), 0, N_LAYERS, objs, B,
                                         s.cuda_stream)
    s.synchronize()
    for l in range(N_LAYERS):
        exp = torch.zeros_like(kv[l])
        for k, d in zip((8, 3, 1, 6), dst_blocks):
            exp[:, d] = kv[l][:, src_block_of[k]]
        assert torch.equal(new_cache[l].view(torch.int16), exp.view(torch.int16)), l
    st = ring.stats()
    assert st["bytes_saved"] == 9 * ENTRY and st["bytes_loaded"] == 4 * ENTRY
    assert st["blocks_asked_for"] == 9 and st["blocks_already_here"] == 2
    assert st["entries_given_away"] == 1 and st["entries_in_use"] == 8
    assert st["lookups_found"] == 4 and st["lookups_missed"] == 2
    ring.close()


def test_objects_spaced_wider_than_an_entry_and_the_error_cases():
    kv = _caches(6)
    cache = _cache_handle(kv)
    ring = kvt_amd.ObjectRing(0, ENTRY, 4, 16)
    s = checkers.side_stream()
    blocks, keys = [4, 17, 9], [key(i) for i in (40, 41, 42)]
    e, new = _save(ring, kv, cache, blocks, keys, s, pad=4096)
    assert new.all()
    for b, idx in zip(blocks, e):
        ring.wait(idx)
        assert np.array_equal(ring.entry(idx), _object_of(kv, b)), b
    back = torch.zeros(3 * (ENTRY + 512), dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    ring.load(e[::-1].copy(), back.data_ptr(), ENTRY + 512, s.cuda_stream)
    s.synchronize()
    host = back.cpu().numpy()
    for i, b in enumerate(blocks[::-1]):
        assert np.array_equal(host[i * (ENTRY + 512):i * (ENTRY + 512) + ENTRY], _object_of(kv, b))
        assert not host[i * (ENTRY + 512) + ENTRY:(i + 1) * (ENTRY + 512)].any()

    e4, new4 = ring.reserve([key(43)])
    assert new4.all()
    small = torch.zeros(ENTRY, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    with pytest.raises(kvt_amd.KvtError) as ex:          # reserved, never written
        ring.load(e4, small.data_ptr(), ENTRY, s.cuda_stream)
    assert "has not been written" in str(ex.value)
    with pytest.raises(kvt_amd.KvtError):                # stride smaller than an entry
        ring.save(e4, small.data_ptr(), ENTRY - 1, s.cuda_stream)
    with pytest.raises(kvt_amd.KvtError) as ex:          # never handed out
        ring.save(np.array([9], dtype=np.uint32), small.data_ptr(), ENTRY, s.cuda_stream)
    assert ex.value.code == 1
    big = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    with pytest.raises(kvt_amd.KvtError) as ex:          # two objects do not fit behind the pointer
        ring.save(np.array([0, 1], dtype=np.uint32), big.data_ptr() + (1 << 20) - ENTRY,
                  1 << 44, s.cuda_stream)
    assert "device buffer" in str(ex.value)
    # the entry that was reserved can still be written by the host and then loaded
    ring.entry(e4[0])[:] = 0x5A
    ring.commit(e4)
    ring.load(e4, small.data_ptr(), ENTRY, s.cuda_stream)
    s.synchronize()
    assert (small == 0x5A).all()
    ring.close()


def test_a_ring_that_wraps_many_times_under_overlapping_saves_and_loads():
    """Entries are reused while transfers are still queued: giving an entry to a new key waits
    for the transfer that uses it, so no object is ever a mix of two blocks."""
    kv = _caches(7)
    cache = _cache_handle(kv)
    ring = kvt_amd.ObjectRing(0, ENTRY, 6, 16)
    s = checkers.side_stream()
    rng = np.random.default_rng(3)
    for step in range(40):
        blocks = rng.permutation(NBLK)[:4].tolist()
        # the key names the block's content here, as a hash would
        keys = [key(b) for b in blocks]
        entries, new = ring.reserve(keys)
        todo = [b for b, n in zip(blocks, new) if n]
        if todo:
            objs = torch.empty(len(todo) * ENTRY, dtype=torch.uint8, device="cuda")
            _plan(todo, todo).pack(cache, 0, N_LAYERS, objs, B, s.cuda_stream)
            ring.save(entries[new], objs.data_ptr(), ENTRY, s.cuda_stream)   # not waited for
        probe = rng.permutation(NBLK)[:6].tolist()
        e, found = ring.lookup([key(b) for b in probe])
        hit = [b for b, f in zip(probe, found) if f]
        if hit:
            back = torch.empty(len(hit) * ENTRY, dtype=torch.uint8, device="cuda")
            ring.load(e[found], back.data_ptr(), ENTRY, s.cuda_stream)
            s.synchronize()
            host = back.cpu().numpy()
            for i, b in enumerate(hit):
                assert np.array_equal(host[i * ENTRY:(i + 1) * ENTRY], _object_of(kv, b)), (step, b)
    ring.close()
