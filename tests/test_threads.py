"""A compiled parser is immutable: many threads may parse with it at once (the
reference runs one sender thread per destination, kvtransfer/src/client.cpp:94-104),
and the error message is per thread. CPU only."""
import threading

import numpy as np

import cases
import kvt_amd
from kvt_amd import workloads


def test_one_parser_many_threads():
    w = workloads.tp_split("flash", 2, 1, 1, n_layers=1, src_pool=600, dst_pool=5000, n_req=24,
                           min_tok=200, max_tok=3000)
    src, dst = w.worker_infos()
    valid, tp_size, tp_rank, pid, kind = kvt_amd.select_parser(w.cache_shape, src, dst)
    parser = kvt_amd.Parser(pid, src, dst, valid, tp_size, tp_rank)
    tasks = w.task_bufs()
    ref = kvt_amd.BlockLists()
    for t in tasks:
        assert parser.parse(t.struct, ref) == 0
    want = ref.tensor(0)
    results, errors = [None] * 8, []

    def work(i):
        try:
            for _ in range(5):
                lists, runs = kvt_amd.BlockLists(), kvt_amd.RunLists()
                for t in tasks:
                    assert parser.parse(t.struct, lists) == 0
                    assert parser.parse_runs(t.struct, runs) == 0
                assert np.array_equal(runs.expand().tensor(0), lists.tensor(0))
                results[i] = lists.tensor(0)
        except Exception as e:      # surfaced below; an exception in a thread is otherwise lost
            errors.append(e)

    threads = [threading.Thread(target=work, args=(i,)) for i in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for r in results:
        assert np.array_equal(r, want)


def test_error_message_is_per_thread():
    case = cases.gen_case("FLASH_PEQD", 1)
    pid, src, dst, valid, tps, tpr, tasks = cases.materialise(case)
    parser = kvt_amd.Parser(pid, src, dst, valid, tps, tpr)
    L = kvt_amd.lib()
    seen = {}

    def failing():
        assert L.kvt_parse_block(parser.h, None, None) != 0
        seen["failing"] = L.kvt_last_error().decode()

    def clean():
        lists = kvt_amd.BlockLists()
        assert parser.parse(tasks[0].struct, lists) in (0, 1)
        seen["clean_before"] = L.kvt_last_error().decode()

    a = threading.Thread(target=failing)
    a.start()
    a.join()
    b = threading.Thread(target=clean)
    b.start()
    b.join()
    assert "null argument" in seen["failing"]
    assert "null argument" not in seen["clean_before"]


def test_object_ring_reservations_of_one_thread_survive_the_others():
    """Eight threads push batches through one small ring (host-only): between a thread's reserve
    and its commit nobody else may be handed its entries, so the tag it wrote is still there."""
    n_entries, batch = 12, 3
    ring = kvt_amd.ObjectRing(-1, 32, n_entries, 16)
    errors, done = [], [0] * 8

    def work(tid):
        try:
            rng = np.random.default_rng(tid)
            for step in range(300):
                ids = rng.integers(0, 40, size=batch)
                keys = [int(i).to_bytes(8, "little") + b"thread%02d" % 0 for i in ids]
                try:
                    entries, new = ring.reserve(keys)
                except kvt_amd.KvtError:
                    continue                  # the others hold everything right now
                mine = sorted({int(e) for e, n in zip(entries, new) if n})
                tag = (tid << 16) | step
                for e in mine:
                    ring.entry(e).view(np.uint32)[0] = tag
                for e in mine:                # (several threads may be asked for the same
                    got = int(ring.entry(e).view(np.uint32)[0])   # block; then the tag is one of theirs)
                    assert (got & 0xFFFF) < 300 and (got >> 16) < 8
                if step % 5 == 4:
                    ring.release(np.array(mine, dtype=np.uint32))
                else:
                    ring.commit(np.array(mine, dtype=np.uint32))
                _, found = ring.lookup(keys)
                done[tid] += int(found.sum())
        except Exception as exc:              # noqa: BLE001
            errors.append((tid, repr(exc)))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    assert sum(done) > 0
    # the index is still consistent: every key found names a distinct entry
    keys = [int(i).to_bytes(8, "little") + b"thread00" for i in range(40)]
    e, found = ring.lookup(keys)
    hit = e[found].tolist()
    assert len(hit) == len(set(hit)) and len(hit) <= n_entries
    ring.close()
