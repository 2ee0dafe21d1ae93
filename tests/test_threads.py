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
