"""A loopback channel with the reference's IChannel surface
(kvtransfer/include/channel.h:59-83: connect / register_data / send_data /
flush / is_active / close), built on the library: register_data makes the
batch's ranges resident as a copy plan, send_data(layer) gathers the layer into
a transfer buffer and scatters it into the destination cache. It is what the
reference's own end-to-end test plugs in as FakeChannel
(kvtransfer/tests/client_step_test.cu:22-50), with the per-range copies replaced
by one pack and one unpack launch per layer.

With `events` (one per layer, recorded by the producer of the layer on its
compute stream) send_data never blocks the host: the dependency is a stream
wait on the library's side stream (the role of CudaEventBarrier + Step in the
reference, kvtransfer/src/step.cpp:49-69)."""
import time

from . import binding
from .ctypes_defs import TP_PEQD


class LoopbackChannel:
    def __init__(self, device, src_cache, dst_cache, src_capacity, dst_capacity):
        self.device = device
        self.src_cache, self.dst_cache = src_cache, dst_cache
        self.src_capacity, self.dst_capacity = list(src_capacity), list(dst_capacity)
        self.plan = self.session = self._buf = None
        self._active = False
        self._stats = {}

    # -- IChannel ---------------------------------------------------------------
    def connect(self, dst_info):
        self.dst_info = dst_info
        self._active = True

    def is_active(self):
        return self._active

    def register_data(self, lists, tp_kind, n_layers, alloc):
        """lists: BlockLists of the batch (borrowed until flush, as in the reference);
        tp_kind: TPKind; alloc(nbytes) -> device buffer for n_layers packed layers."""
        if not self._active:
            raise RuntimeError("register_data on a channel that is not connected")
        t0 = time.perf_counter()
        if tp_kind == TP_PEQD:
            lists.merge()                    # merge_interval + erase, tcp_channel.cpp:376-392
        for t in range(lists.num_tensors()):
            rc, bad = binding.validate_bounds(lists.tensor(t), self.dst_capacity[t], 1)
            if rc != 0:
                raise binding.KvtError(rc, "rejected invalid copy metadata (range %d)" % bad)
        if tp_kind == TP_PEQD:
            source = lists
        else:   # per-token ranges of a TP remap: fold them back into strided runs
            source = binding.RunLists.compress(lists)
        self.plan = binding.Plan(self.device, source, self.src_capacity, self.dst_capacity)
        self.stride = self.plan.layer_bytes
        self._buf = alloc(max(1, n_layers * self.stride))
        self.session = binding.Session(self.plan, self.src_cache, self._buf, self.stride)
        self._stats = {"sb_num": sum(len(lists.tensor(t)) for t in range(lists.num_tensors())),
                       "sb_size_total": sum(self.plan.tensor_bytes(t)
                                            for t in range(lists.num_tensors())),
                       "register_us": int((time.perf_counter() - t0) * 1e6), "layers_sent": 0}

    def send_data(self, layer_index, compute_stream=None):
        """Packs the layer once everything queued on compute_stream so far has run,
        then unpacks it into the destination cache. Does not block the host."""
        self.session.save_layer(layer_index, compute_stream)
        side = self.session.side_stream
        self.plan.unpack(self.dst_cache, layer_index, 1, binding._ptr(self._buf) +
                         layer_index * self.stride, self.stride, side)
        self._stats["layers_sent"] += 1

    def flush(self):
        """Blocks until everything sent has landed; returns the reference-style 'k=v,' string."""
        binding.check(binding.lib().kvt_stream_synchronize(self.session.side_stream))
        out = "".join("%s=%s," % kv for kv in sorted(self._stats.items()))
        return out

    def close(self):
        for obj in (self.session, self.plan):
            if obj is not None:
                obj.close()
        self.session = self.plan = self._buf = None
        self._active = False
