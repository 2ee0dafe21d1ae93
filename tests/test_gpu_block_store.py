"""kvt_amd.block_store.FileBlockStore against what the reference's FileBackend does with the
same (blkid, blkhash) lists (blade_kvt/hybrid_connector/file_backend.py:215-285): a saved
block's file holds kvcache[:, blkid] of every layer, a ready block is not written again, and
loading puts the bytes into whatever block id the request was given — also by a second store
that only has the directory. Needs a real MI355X."""
import os

import numpy as np
import pytest

from kvt_amd.block_store import FileBlockStore

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

N_LAYERS, NBLK, BS, H, D = 3, 40, 16, 4, 32


def _caches(seed, zeros=False):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    kv = {}
    for l in range(N_LAYERS):
        t = torch.randn((2, NBLK, BS, H, D), generator=g, device="cuda").to(torch.bfloat16)
        kv["model.layers.%d.self_attn.attn" % l] = torch.zeros_like(t) if zeros else t
    torch.cuda.synchronize()
    return kv


def _expected_file(kv, blkid):
    return torch.stack([t[:, blkid] for t in kv.values()]).contiguous().view(torch.uint8) \
        .reshape(-1).cpu().numpy()


def test_save_skip_and_load_like_the_file_backend(tmp_path):
    kv = _caches(1)
    store = FileBlockStore(str(tmp_path), ring_entries=8)
    store.register_kv_caches(kv)
    blks = [(5, "1_2_3"), (17, "1_2_3_4_5"), (2, "9_9"), (30, "7")]
    assert store.save_blocks(blks) == 4
    for blkid, blkhash in blks:
        blkdir = tmp_path / blkhash
        assert (blkdir / "ready").is_file()
        data = np.fromfile(blkdir / "0.data", dtype=np.uint8)
        assert np.array_equal(data, _expected_file(kv, blkid)), blkhash
    # ready blocks are skipped, whatever block id they come with; a new one is written
    stamp = {h: os.stat(tmp_path / h / "0.data").st_mtime_ns for _, h in blks}
    assert store.save_blocks([(6, "1_2_3"), (11, "5_5_5"), (11, "5_5_5")]) == 1
    assert stamp == {h: os.stat(tmp_path / h / "0.data").st_mtime_ns for _, h in blks}
    assert np.array_equal(np.fromfile(tmp_path / "5_5_5" / "0.data", dtype=np.uint8),
                          _expected_file(kv, 11))
    # more blocks than the ring has entries: batches of 8, the oldest entries are reused
    many = [(b, "many_%d" % b) for b in range(20)]
    assert store.save_blocks(many) == 20
    for b, h in many:
        assert np.array_equal(np.fromfile(tmp_path / h / "0.data", dtype=np.uint8),
                              _expected_file(kv, b))

    # the same store loads into other block ids of its own caches (some from the ring, the
    # early ones from their files)
    before = {n: t.clone() for n, t in kv.items()}
    store.load_blocks([(33, "1_2_3"), (34, "many_19"), (35, "9_9")])
    for n, t in kv.items():
        exp = before[n].clone()
        exp[:, 33], exp[:, 34], exp[:, 35] = before[n][:, 5], before[n][:, 19], before[n][:, 2]
        assert torch.equal(t.view(torch.int16), exp.view(torch.int16)), n
    store.close()

    # a second instance that has nothing but the directory (a decode node, or a restart)
    fresh = _caches(0, zeros=True)
    other = FileBlockStore(str(tmp_path), ring_entries=4)
    other.register_kv_caches(fresh)
    want = [(0, "7"), (1, "1_2_3_4_5"), (2, "many_3"), (3, "many_4"), (4, "many_5"), (9, "7")]
    other.load_blocks(want)
    src_of = {"7": 30, "1_2_3_4_5": 17, "many_3": 3, "many_4": 4, "many_5": 5}
    for (n, t), (_, s) in zip(fresh.items(), before.items()):
        exp = torch.zeros_like(t)
        for blkid, h in want:
            exp[:, blkid] = s[:, src_of[h]]
        assert torch.equal(t.view(torch.int16), exp.view(torch.int16)), n
    with pytest.raises(KeyError):
        other.load_blocks([(5, "never_saved")])
    other.close()


def test_layer_wise_save_while_the_layers_are_being_produced(tmp_path):
    """async_save_kv_layer's shape: each layer is handed over right after the kernel that
    writes it has been queued; a block is ready only after the last layer."""
    kv = _caches(3, zeros=True)
    final = _caches(3)
    store = FileBlockStore(str(tmp_path), ring_entries=8)
    store.register_kv_caches(kv)
    blks = [(4, "a_1"), (21, "a_2"), (8, "a_3")]
    names = list(kv)
    for l, name in enumerate(names):
        kv[name].copy_(final[name])                 # "the forward pass" fills layer l on torch's stream
        done = store.save_kv_layer(l, blks)
        if l < len(names) - 1:
            assert done == 0 and not (tmp_path / "a_1" / "ready").exists()
    assert done == 3
    for blkid, blkhash in blks:
        assert (tmp_path / blkhash / "ready").is_file()
        assert np.array_equal(np.fromfile(tmp_path / blkhash / "0.data", dtype=np.uint8),
                              _expected_file(final, blkid)), blkhash
    # a later step with the same blocks has nothing to do
    for l in range(len(names)):
        assert store.save_kv_layer(l, blks) == 0
    store.close()


def test_abandoned_layer_wise_steps_give_their_ring_entries_back(tmp_path):
    """A step that never reaches its last layer (an aborted forward pass, a failing pack) must
    not keep its entries claimed: after more abandoned steps than the ring has entries the
    next complete step still finds room, and what it writes is exact."""
    kv = _caches(5)
    store = FileBlockStore(str(tmp_path), ring_entries=4)
    store.register_kv_caches(kv)
    names = list(kv)
    for attempt in range(6):                       # 6 x 3 blocks > 4 entries
        blks = [(b, "gone_%d_%d" % (attempt, b)) for b in (1, 2, 3)]
        assert store.save_kv_layer(0, blks) == 0   # layer 0 only: the step is then dropped
    # a pack that fails mid-step settles its claims too
    blks = [(7, "fail_7"), (8, "fail_8")]
    assert store.save_kv_layer(0, blks) == 0
    with pytest.raises(Exception):
        store.save_kv_layer(len(names) + 5, blks)  # no such layer: the pack is refused
    assert store._step is None
    stats = store._ring.stats()
    assert stats["entries_in_use"] == 0, stats
    blks = [(9, "kept_9"), (10, "kept_10"), (11, "kept_11"), (12, "kept_12")]
    for l in range(len(names)):
        done = store.save_kv_layer(l, blks)
    assert done == 4
    for blkid, blkhash in blks:
        assert np.array_equal(np.fromfile(tmp_path / blkhash / "0.data", dtype=np.uint8),
                              _expected_file(kv, blkid)), blkhash
    assert not (tmp_path / "gone_0_1").exists() and not (tmp_path / "fail_7").exists()
    store.close()
