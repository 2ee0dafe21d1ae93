"""The data plane of the reference's file store on the GPU path.

FileBackend (reference: blade_kvt/hybrid_connector/file_backend.py) keeps, per
block hash, a directory with one ``torch.save(kvcache[:, blkid])`` per layer and
a ``ready`` marker (:52-60, :258-285); it skips blocks that are ready and loads a
ready block back with ``kvcache[:, blkid] = cpublk.to(device)`` per layer
(:215-233). Every block costs ``2 * n_layers`` small copies there. Here a batch
of blocks is one pack launch (all layers of a block into one object), DMA copies
into the pinned ring, and one file per block; loading is the mirror. Same
``(blkid, blkhash)`` lists, same ``ready`` marker, same directory per hash; the
file inside holds the raw bytes of ``stack([kvcache_l[:, blkid] for l in layers])``
instead of one pickle per layer.

What is mirrored is register_kv_caches / the save and load of block lists; the
scheduler side of the backend (prefix matching, operation plans) is not part of
this path."""
import hashlib
import os

import numpy as np

from . import binding
from .ctypes_defs import SHAPE_FLASH, make_worker_info


def _blk_ready(path):
    return os.path.isdir(path) and os.path.isfile(os.path.join(path, "ready"))


class FileBlockStore:
    def __init__(self, cachedir, device=0, rank=0, ring_entries=256):
        self._dir, self._device, self._rank, self._ring_entries = cachedir, device, rank, ring_entries
        self._kv = None
        self._step = None

    def register_kv_caches(self, kv_caches):
        """kv_caches: {layer name: tensor [2, num_blocks, block_size, heads, head_dim]} on the
        GPU, contiguous, all of one shape and dtype (what FileBackend asserts on load, :226-231)."""
        import torch
        self._torch = torch
        layers = list(kv_caches.values())
        first = layers[0]
        assert first.dim() == 5 and first.size(0) == 2
        for t in layers:
            assert t.shape == first.shape and t.dtype == first.dtype and t.is_contiguous()
        self._kv = layers
        self._nblk = first.size(1)
        self._obj = 2 * first[0, 0].numel() * first.element_size()       # kvcache[:, b], bytes
        self._entry = self._obj * len(layers)
        self._info = make_worker_info(block_sizes=[self._obj], token_sizes=[self._obj // first.size(2)],
                                      layer_num_blocks=self._nblk, num_layers=len(layers))
        cap = [self._obj * self._nblk]
        self._cap = cap
        self._cache = binding.Cache(self._device, [[t.view(torch.uint8).reshape(-1)] for t in layers], cap)
        self._ring = binding.ObjectRing(self._device, self._entry, self._ring_entries, 32)
        self._stream = torch.cuda.Stream()

    @staticmethod
    def _key(blkhash):
        return hashlib.sha256(blkhash.encode()).digest()

    def _plan(self, blkids):
        ids = np.asarray(blkids, dtype=np.uint32)
        lists, ob = binding.block_object_lists(SHAPE_FLASH, self._info, self._info, ids, ids)
        assert ob == self._obj
        return binding.Plan(self._device, lists, self._cap, self._cap, objects=(ob, self._entry))

    def _path(self, blkhash):
        blkdir = os.path.join(self._dir, blkhash)
        return blkdir, os.path.join(blkdir, "%d.data" % self._rank)

    def save_blocks(self, blks):
        """blks: [(blkid, blkhash)]. Blocks whose hash is ready are skipped (file_backend.py:
        266-270). -> number of blocks written."""
        torch = self._torch
        todo = []
        seen = set()
        for blkid, blkhash in blks:
            if blkhash in seen or _blk_ready(self._path(blkhash)[0]):
                continue
            seen.add(blkhash)
            todo.append((blkid, blkhash))
        written = 0
        for at in range(0, len(todo), self._ring_entries):
            part = todo[at:at + self._ring_entries]
            entries, new = self._ring.reserve([self._key(h) for _, h in part])
            fresh = [b for (b, _), n in zip(part, new) if n]
            if fresh:
                try:
                    objs = torch.empty(len(fresh) * self._entry, dtype=torch.uint8, device="cuda")
                    self._stream.wait_stream(torch.cuda.current_stream())
                    plan = self._plan(fresh)
                    plan.pack(self._cache, 0, len(self._kv), objs, self._obj, self._stream.cuda_stream)
                    self._ring.save(entries[new], objs.data_ptr(), self._entry,
                                    self._stream.cuda_stream)
                except Exception:
                    self._ring.release(entries[new])    # every "new" answer is settled exactly once
                    raise
                self._stream.synchronize()
                plan.close()
            for (blkid, blkhash), idx in zip(part, entries):
                blkdir, datapath = self._path(blkhash)
                os.makedirs(blkdir, exist_ok=True)
                self._ring.wait(idx)
                self._ring.entry(idx).tofile(datapath)
                with open(os.path.join(blkdir, "ready"), "w"):
                    pass
                written += 1
        return written

    def save_kv_layer(self, layer_idx, blks):
        """The layer-wise form, called once per layer while the forward pass runs (FileBackend.
        async_save_kv_layer / _save_layer, file_backend.py:258-300): layer `layer_idx` of the
        not-yet-ready blocks is packed behind the work queued on torch's current stream; after
        the last layer the objects are written out and marked ready (:282-283). One batch (at
        most ring_entries new blocks) is in flight at a time. -> blocks written by this call."""
        torch = self._torch
        n_layers = len(self._kv)
        if layer_idx == 0:
            self._abandon_step()       # a step that never reached its last layer
            todo, seen = [], set()
            for blkid, blkhash in blks:
                if blkhash not in seen and not _blk_ready(self._path(blkhash)[0]):
                    seen.add(blkhash)
                    todo.append((blkid, blkhash))
            if len(todo) > self._ring_entries:
                raise ValueError("more new blocks in one step than the ring has entries")
            if todo:
                entries, new = self._ring.reserve([self._key(h) for _, h in todo])
                # only the entries this call was given (new) are written and settled by it; the
                # others are being filled, or were filled, by whoever reserved them first
                fresh = [b for (b, _), n in zip(todo, new) if n]
                try:
                    objs = torch.empty(len(fresh) * self._entry, dtype=torch.uint8, device="cuda")
                    plan = self._plan(fresh) if fresh else None
                except Exception:
                    self._ring.release(entries[new])
                    raise
                self._step = (todo, entries, new, objs, plan)
        if self._step is None:
            return 0
        todo, entries, new, objs, plan = self._step
        try:
            if plan is not None:
                self._stream.wait_stream(torch.cuda.current_stream())  # the layer has been computed
                plan.pack(self._cache, layer_idx, 1, objs[layer_idx * self._obj:], self._obj,
                          self._stream.cuda_stream)
            if layer_idx != n_layers - 1:
                return 0
            if plan is not None:
                self._ring.save(entries[new], objs.data_ptr(), self._entry, self._stream.cuda_stream)
                new = np.zeros_like(new)          # settled: nothing left to give back on failure
                self._step = (todo, entries, new, objs, plan)
                self._stream.synchronize()
            for (blkid, blkhash), idx in zip(todo, entries):
                blkdir, datapath = self._path(blkhash)
                os.makedirs(blkdir, exist_ok=True)
                self._ring.wait(idx)
                self._ring.entry(idx).tofile(datapath)
                with open(os.path.join(blkdir, "ready"), "w"):
                    pass
        except Exception:
            self._abandon_step()
            raise
        if plan is not None:
            plan.close()
        self._step = None
        return len(todo)

    def _abandon_step(self):
        """Gives back what an unfinished layer-wise step holds: its claims on ring entries (an
        entry that stays claimed is never handed out again) and its plan."""
        if self._step is None:
            return
        todo, entries, new, objs, plan = self._step
        self._step = None
        self._stream.synchronize()          # packs of the abandoned step still write to objs
        if new.any():
            self._ring.release(entries[new])
        if plan is not None:
            plan.close()

    def load_blocks(self, blks):
        """blks: [(blkid, blkhash)]: every block must be ready (file_backend.py:219-221); its
        bytes go into block `blkid` of every registered layer."""
        torch = self._torch
        for at in range(0, len(blks), self._ring_entries):
            part = blks[at:at + self._ring_entries]
            keys = [self._key(h) for _, h in part]
            entries, found = self._ring.lookup(keys)
            missing = [i for i, f in enumerate(found) if not f]
            if missing:
                for i in missing:
                    if not _blk_ready(self._path(part[i][1])[0]):
                        raise KeyError(part[i][1])
                # every entry this batch refers to is kept by the reservation
                entries, new = self._ring.reserve(keys)
                filled = []
                try:
                    for i, (idx, n) in enumerate(zip(entries, new)):
                        if n:
                            data = np.fromfile(self._path(part[i][1])[1], dtype=np.uint8)
                            assert data.size == self._entry
                            self._ring.entry(idx)[:] = data
                            filled.append(idx)
                except Exception:
                    self._ring.release(entries[new])
                    raise
                self._ring.commit(np.asarray(filled, dtype=np.uint32))
            objs = torch.empty(len(part) * self._entry, dtype=torch.uint8, device="cuda")
            self._stream.wait_stream(torch.cuda.current_stream())
            self._ring.load(entries, objs.data_ptr(), self._entry, self._stream.cuda_stream,
                            keys=keys)
            plan = self._plan([b for b, _ in part])
            plan.unpack(self._cache, 0, len(self._kv), objs, self._obj, self._stream.cuda_stream)
            self._stream.synchronize()
            plan.close()

    def close(self):
        if self._kv is not None:
            self._abandon_step()
            self._ring.close()
            self._cache.close()
            self._kv = None
