"""The index of the pinned object ring (kvt_object_ring_*), on a ring created without a
device: which keys count as new, which entries they get, what is given away when the ring is
full. Checked case by case and against a small Python model on random traffic. The GPU side
(save / load through DMA copies) is in tests/test_gpu_object_ring.py. CPU only."""
import ctypes as C

import numpy as np
import pytest

import kvt_amd

NONE = -1          # KVT_DEVICE_NONE


def key(i):
    return int(i).to_bytes(8, "little") + b"blockkey"


def ring(n_entries=4, entry_bytes=64):
    return kvt_amd.ObjectRing(NONE, entry_bytes, n_entries, 16)


def test_new_keys_get_neighbouring_entries_and_are_found_once_written():
    r = ring(8)
    e, new = r.reserve([key(i) for i in range(5)])
    assert e.tolist() == [0, 1, 2, 3, 4] and new.all()
    _, found = r.lookup([key(i) for i in range(5)])
    assert not found.any()                      # reserved, not written
    r.commit(e[:3])
    e2, found = r.lookup([key(i) for i in range(5)])
    assert found.tolist() == [True, True, True, False, False] and e2[:3].tolist() == [0, 1, 2]
    # a second reservation: written blocks are skipped (the reference's _blk_ready), the two
    # that were never written are asked for again, in their old entries
    e3, new = r.reserve([key(i) for i in range(5)])
    assert e3.tolist() == [0, 1, 2, 3, 4] and new.tolist() == [False, False, False, True, True]


def test_a_key_repeated_inside_a_batch_is_asked_for_once():
    r = ring(8)
    e, new = r.reserve([key(1), key(2), key(1), key(1), key(3)])
    assert e.tolist() == [0, 1, 0, 0, 2]
    assert new.tolist() == [True, True, False, False, True]
    e, new = r.reserve([key(1), key(1)])        # still unwritten: asked again, once
    assert e.tolist() == [0, 0] and new.tolist() == [True, False]


def test_a_full_ring_gives_its_oldest_entries_to_new_keys():
    r = ring(4)
    e, _ = r.reserve([key(i) for i in range(4)])
    r.commit(e)
    e, new = r.reserve([key(10), key(11)])
    assert e.tolist() == [0, 1] and new.all()
    _, found = r.lookup([key(0), key(1), key(2), key(3), key(10)])
    assert found.tolist() == [False, False, True, True, False]


def test_entries_a_batch_refers_to_are_not_given_away_by_it():
    r = ring(4)
    e, _ = r.reserve([key(i) for i in range(4)])
    r.commit(e)
    # key 0 is stored in entry 0, the next entry in ring order: the three new keys go around it
    e, new = r.reserve([key(20), key(0), key(21), key(22)])
    assert e.tolist() == [1, 0, 2, 3] and new.tolist() == [True, False, True, True]
    _, found = r.lookup([key(0), key(1), key(2), key(3)])
    assert found.tolist() == [True, False, False, False]


def test_a_batch_larger_than_the_ring_is_refused_but_repeats_do_not_count():
    r = ring(4)
    with pytest.raises(kvt_amd.KvtError) as ex:
        r.reserve([key(i) for i in range(5)])
    assert ex.value.code == 3 and "more new blocks" in str(ex.value)
    e, new = r.reserve([key(i % 4) for i in range(12)])
    assert e.tolist() == [0, 1, 2, 3] * 3 and new.tolist() == [True] * 4 + [False] * 8
    r.commit(e[:1])
    with pytest.raises(kvt_amd.KvtError):       # one stored block referred to + four new ones
        r.reserve([key(0), key(30), key(31), key(32), key(33)])


def test_a_reservation_stays_until_it_is_written_or_released():
    """Between one thread's reserve and its save another thread's batch must not be given the
    same entries: what somebody has yet to write is not given away."""
    r = ring(4)
    mine, _ = r.reserve([key(1), key(2)])               # not written yet
    theirs, new = r.reserve([key(3), key(4)])
    assert sorted(mine.tolist() + theirs.tolist()) == [0, 1, 2, 3] and new.all()
    with pytest.raises(kvt_amd.KvtError):                # all four entries are spoken for
        r.reserve([key(5)])
    r.commit(theirs)
    e, _ = r.reserve([key(5)])                           # a written entry may go
    assert e.tolist() == [int(theirs[0])]
    r.release(mine[:1])                                  # key 1 will not be written after all
    _, found = r.lookup([key(1)])
    assert not found.any()
    e, new = r.reserve([key(1)])                         # forgotten: a fresh reservation,
    assert new.all() and e.tolist() == [int(theirs[1])]   # in the next entry in ring order
    r.commit(e)
    r.release(e)                                         # written and nobody waiting: left alone
    _, found = r.lookup([key(1)])
    assert found.all()
    with pytest.raises(kvt_amd.KvtError):
        r.release(np.array([4], dtype=np.uint32))


def test_two_callers_asked_for_the_same_block():
    r = ring(2)
    a, new_a = r.reserve([key(7)])
    b, new_b = r.reserve([key(7)])                       # the first has not written it yet
    assert a.tolist() == b.tolist() == [0] and new_a.all() and new_b.all()
    r.release(a)                                         # the first gives up: the second still holds it
    e, new = r.reserve([key(8), key(9)][:1])
    assert e.tolist() == [1] and new.all()
    with pytest.raises(kvt_amd.KvtError):                # entry 0 is still somebody's
        r.reserve([key(9)])
    r.commit(b)
    _, found = r.lookup([key(7)])
    assert found.all()
    # and the other way round: written by one while the other is still at it -> stays put
    r2 = ring(1)
    a, _ = r2.reserve([key(1)])
    b, _ = r2.reserve([key(1)])
    r2.commit(a)
    with pytest.raises(kvt_amd.KvtError):
        r2.reserve([key(2)])
    r2.commit(b)
    e, new = r2.reserve([key(2)])
    assert e.tolist() == [0] and new.all()


def test_entries_are_separate_pieces_of_host_memory():
    r = ring(3, entry_bytes=96)
    e, _ = r.reserve([key(1), key(2), key(3)])
    for i, idx in enumerate(e):
        r.entry(idx)[:] = i + 1
    for i, idx in enumerate(e):
        assert (r.entry(idx) == i + 1).all()
    base = r.entry(0).ctypes.data
    assert [r.entry(i).ctypes.data - base for i in range(3)] == [0, 96, 192]
    with pytest.raises(IndexError):
        r.entry(3)


def test_bad_arguments_and_no_device():
    lib = kvt_amd.lib()
    h = C.c_void_p()
    for args in ((NONE, 0, 4, 16), (NONE, 64, 0, 16), (NONE, 64, 4, 0), (NONE, 64, 4, 257),
                 (NONE, 1 << 63, 4, 16)):
        assert lib.kvt_object_ring_create(*args, C.byref(h)) != 0, args
    r = ring(4)
    e, _ = r.reserve([key(1)])
    with pytest.raises(kvt_amd.KvtError) as ex:            # never handed out
        r.commit(np.array([3], dtype=np.uint32))
    assert ex.value.code == 1
    with pytest.raises(kvt_amd.KvtError) as ex:
        r.commit(np.array([4], dtype=np.uint32))
    assert ex.value.code == 1
    buf = np.zeros(64, dtype=np.uint8)
    with pytest.raises(kvt_amd.KvtError) as ex:
        r.save(e, buf.ctypes.data, 64)
    assert ex.value.code == 6                               # no device: there is no CPU copy path
    with pytest.raises(kvt_amd.KvtError) as ex:
        r.load(e, buf.ctypes.data, 64)
    assert ex.value.code == 6
    r.wait(0)
    assert lib.kvt_object_ring_wait(r.h, 4) != 0
    assert lib.kvt_object_ring_reserve(None, None, 0, None, None) != 0
    r.close()
    r.close()


class Model:
    """The ring's rules, restated."""

    def __init__(self, n):
        self.n, self.handed_out = n, 0
        self.key, self.saved, self.claims, self.index = [None] * n, [False] * n, [0] * n, {}

    def _may_go(self, idx, touched):
        return idx not in touched and self.claims[idx] == 0

    def reserve(self, keys):
        touched = {self.index[k] for k in keys if k in self.index}
        fresh = {k for k in keys if k not in self.index}
        if len(fresh) > sum(self._may_go(i, touched) for i in range(self.n)):
            return None
        flagged, out = set(), []
        for k in keys:
            if k in self.index:
                idx = self.index[k]
                new = (not self.saved[idx]) and idx not in flagged
                if new:
                    self.claims[idx] += 1
            else:
                while True:
                    idx = self.handed_out % self.n
                    self.handed_out += 1
                    if self._may_go(idx, touched):
                        break
                if self.key[idx] is not None:
                    del self.index[self.key[idx]]
                self.key[idx], self.saved[idx], self.claims[idx], self.index[k] = k, False, 1, idx
                touched.add(idx)
                new = True
            if new:
                flagged.add(idx)
            out.append((idx, new))
        return out

    def commit(self, entries):
        for idx in entries:
            self.saved[idx] = True
            self.claims[idx] = max(0, self.claims[idx] - 1)

    def release(self, entries):
        for idx in entries:
            if self.key[idx] is not None and self.claims[idx] > 0:
                self.claims[idx] -= 1
                if self.claims[idx] == 0 and not self.saved[idx]:
                    del self.index[self.key[idx]]
                    self.key[idx] = None

    def lookup(self, keys):
        return [(k in self.index and self.saved[self.index[k]]) for k in keys]


@pytest.mark.parametrize("seed", range(6))
def test_random_traffic_against_the_model(seed):
    rng = np.random.default_rng(seed)
    n = int(rng.integers(1, 12))
    r, m = ring(n), Model(n)
    universe = [key(i) for i in range(3 * n + 2)]
    for step in range(300):
        keys = [universe[int(i)] for i in rng.integers(0, len(universe), size=int(rng.integers(0, 2 * n + 2)))]
        want = m.reserve(keys)
        if want is None:
            with pytest.raises(kvt_amd.KvtError):
                r.reserve(keys)
            continue
        e, new = r.reserve(keys)
        assert list(zip(e.tolist(), new.tolist())) == want, (seed, step)
        if len(keys) and rng.random() < 0.8:              # write some of what was asked for
            todo = sorted({idx for idx, is_new in want if is_new and rng.random() < 0.7})
            r.commit(np.array(todo, dtype=np.uint32))
            m.commit(todo)
            rest = sorted({idx for idx, is_new in want if is_new} - set(todo))
            if rest and rng.random() < 0.6:               # give up what was not written
                r.release(np.array(rest, dtype=np.uint32))
                m.release(rest)
        if rng.random() < 0.2:                            # stray releases change nothing they should not
            drop = [int(i) for i in rng.integers(0, n, size=int(rng.integers(0, n + 1)))]
            r.release(np.array(drop, dtype=np.uint32))
            m.release(drop)
        probe = [universe[int(i)] for i in rng.integers(0, len(universe), size=5)]
        e, found = r.lookup(probe)
        assert found.tolist() == m.lookup(probe)
        assert all(m.index[k] == int(idx) for k, idx, f in zip(probe, e, found) if f)


def test_counters():
    r = ring(4)
    e, _ = r.reserve([key(1), key(2), key(1)])
    r.commit(e[:2])
    r.reserve([key(1), key(3)])
    r.lookup([key(1), key(2), key(3), key(9)])
    e, _ = r.reserve([key(4), key(5)])          # entry 3, then key 1's entry makes room
    st = r.stats()
    assert st == {"blocks_asked_for": 5, "blocks_already_here": 2, "entries_given_away": 1,
                  "lookups_found": 2, "lookups_missed": 2, "bytes_saved": 0, "bytes_loaded": 0,
                  "entries_in_use": 4}
