"""Host-side flow of one send step, mirroring KvSendStub::TaskContext::do_task
(reference: kvtransfer/src/tx_stub.cpp:158-263): pick the parser for the
destination, run ParseBlock for every request of the batch into one range list
per cache tensor, merge when the TP relation is P==D (what register_data does,
kvtransfer/src/tcp_channel.cpp:376-392) and make the result resident on the GPU
as a copy plan."""
from . import binding
from .ctypes_defs import TP_PEQD


class Sender:
    """What TaskContext keeps per destination (refresh_dst_info, kvtransfer/src/tx_stub.cpp:
    417-591): the valid ranks, this rank's place among them, the TP relation and the parser,
    chosen and compiled ONCE; every batch for that destination then only parses."""

    def __init__(self, cache_shape, src, dst, fp8=False, pad=True):
        valid, tp_size, tp_rank, parser_id, self.tp_kind = binding.select_parser(cache_shape, src, dst)
        self.parser = binding.Parser(parser_id, src, dst, valid, tp_size, tp_rank, fp8=fp8, pad=pad)

    def parse(self, task_bufs):
        """-> BlockLists of the batch, merged when the TP relation is P==D. Raises KvtError on
        the first failing request."""
        lists = binding.BlockLists()
        for t in task_bufs:
            binding.check(self.parser.parse(t.struct, lists))
        if self.tp_kind == TP_PEQD:
            lists.merge()
        return lists

    def parse_runs(self, task_bufs):
        """-> RunLists: the same ranges in closed form (one run per block segment), never merged."""
        runs = binding.RunLists()
        for t in task_bufs:
            binding.check(self.parser.parse_runs(t.struct, runs))
        return runs

    def close(self):
        self.parser.close()


def parse_batch(cache_shape, src, dst, task_bufs, fp8=False, pad=True):
    """-> (BlockLists, tp_kind). Raises KvtError on the first failing request."""
    sender = Sender(cache_shape, src, dst, fp8=fp8, pad=pad)
    try:
        return sender.parse(task_bufs), sender.tp_kind
    finally:
        sender.close()


def build_plan(workload, device=0, chunk_bytes=0):
    """Workload -> (Plan, BlockLists). The lists stay valid for wire metadata."""
    src, dst = workload.worker_infos()
    lists, _ = parse_batch(workload.cache_shape, src, dst, workload.task_bufs())
    plan = binding.Plan(device, lists, workload.capacities("src"), workload.capacities("dst"),
                        xform=workload.xform, chunk_bytes=chunk_bytes)
    return plan, lists


def parse_batch_runs(cache_shape, src, dst, task_bufs, fp8=False, pad=True):
    """-> (RunLists, tp_kind): the same ranges in closed form (one run per block segment).
    Runs are never merged; for P==D use parse_batch()."""
    sender = Sender(cache_shape, src, dst, fp8=fp8, pad=pad)
    try:
        return sender.parse_runs(task_bufs), sender.tp_kind
    finally:
        sender.close()


def build_plan_runs(workload, device=0, chunk_bytes=0):
    """Workload -> (Plan whose per-token arithmetic runs on the device, RunLists). A workload
    whose receiver holds fp8 (notes["fp8"]) is parsed in that mode and packs converting."""
    src, dst = workload.worker_infos()
    fp8 = bool(workload.notes.get("fp8"))
    runs, _ = parse_batch_runs(workload.cache_shape, src, dst, workload.task_bufs(), fp8=fp8)
    plan = binding.Plan(device, runs, workload.capacities("src"), workload.capacities("dst"),
                        chunk_bytes=chunk_bytes, bf16_to_fp8=fp8)
    return plan, runs
