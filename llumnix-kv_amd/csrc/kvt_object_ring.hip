// A ring of store objects in pinned host memory, found by block hash: the
// staging tier between the paged cache on the GPU and a KV store behind it.
// The reference's file store keeps one object per (block hash, layer), skips a
// block whose hash is already stored and loads by hash
// (blade_kvt/hybrid_connector/file_backend.py:215-285); here an entry holds one
// block of all layers (what one pack launch of an object plan produces per
// block), entries are handed out in ring order so that the new blocks of a
// batch sit side by side and cross PCIe as one or two large DMA copies, and the
// oldest entries make room for new ones.
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "kvt_runtime.h"

using namespace kvt;

namespace {

// One event per save / load call, shared by the entries it touched.
struct Transfer {
  hipEvent_t done = nullptr;
  ~Transfer() {
    if (done) (void)hipEventDestroy(done);
  }
};

struct Entry {
  std::string key;                     // empty: never used
  bool saved = false;                  // its bytes have been written (or the write is queued)
  uint32_t claims = 0;                 // callers that were asked for the block's bytes and have
                                       // neither written nor released yet; the entry stays put
  uint64_t touched = 0;                // id of the last reserve call that referred to it
  uint64_t flagged = 0;                // id of the last reserve call that reported it as new
  std::shared_ptr<Transfer> pending;   // last transfer that reads or writes the entry
};

}  // namespace

struct kvt_object_ring {
  int device = KVT_DEVICE_NONE;
  uint64_t entry_bytes = 0;
  uint32_t n_entries = 0, key_bytes = 0;
  uint8_t* arena = nullptr;
  hipStream_t copy = nullptr;
  hipEvent_t fence = nullptr;
  // the kernel route of a transfer that is many short pieces: range metadata (3 int64 per
  // piece) on the device and in pinned memory, in use until `meta_free` has completed
  int64_t* meta_dev = nullptr;
  int64_t* meta_host = nullptr;
  hipEvent_t meta_free = nullptr;
  bool meta_used = false;
  std::mutex mu;
  uint64_t handed_out = 0;   // entries assigned so far; the next one is handed_out % n_entries
  uint64_t calls = 0;
  std::vector<Entry> entries;
  std::unordered_map<std::string, uint32_t> index;
  kvt_object_ring_counters stats{};   // under mu
};

namespace {

int wait_entry(Entry& e) {
  if (e.pending) {
    KVT_HIP(hipEventSynchronize(e.pending->done));
    e.pending.reset();
  }
  return KVT_OK;
}

// Runs of entries that are neighbours in the arena and in the device buffer: one copy each.
template <class Fn>
int for_runs(const kvt_object_ring* r, const uint32_t* entries, uint32_t n, uint64_t dev_stride,
             Fn fn) {
  for (uint32_t i = 0; i < n;) {
    uint32_t j = i + 1;
    if (dev_stride == r->entry_bytes)
      while (j < n && entries[j] == entries[j - 1] + 1) ++j;
    if (int rc = fn(i, j - i)) return rc;
    i = j;
  }
  return KVT_OK;
}

int check_entries(const kvt_object_ring* r, const uint32_t* entries, uint32_t n, const char* who) {
  for (uint32_t i = 0; i < n; ++i)
    if (entries[i] >= r->n_entries || r->entries[entries[i]].key.empty())
      return fail(KVT_ERR_OUT_OF_RANGE, std::string(who) + ": entry index not in use");
  return KVT_OK;
}

}  // namespace

extern "C" {

int kvt_object_ring_create(int device, uint64_t entry_bytes, uint32_t n_entries,
                           uint32_t key_bytes, kvt_object_ring** out) {
  return guarded([&]() -> int {
    if (!out || entry_bytes == 0 || n_entries == 0 || key_bytes == 0 || key_bytes > 256)
      return fail(KVT_ERR_INVALID, "kvt_object_ring_create: bad argument");
    uint64_t total = 0;
    if (__builtin_mul_overflow(entry_bytes, static_cast<uint64_t>(n_entries), &total))
      return fail(KVT_ERR_OVERFLOW, "kvt_object_ring_create: ring size overflows");
    std::unique_ptr<kvt_object_ring, void (*)(kvt_object_ring*)> r(new kvt_object_ring(),
                                                                   kvt_object_ring_destroy);
    r->device = device;
    r->entry_bytes = entry_bytes;
    r->n_entries = n_entries;
    r->key_bytes = key_bytes;
    r->entries.resize(n_entries);
    if (device == KVT_DEVICE_NONE) {
      // index only (tests, or a store that fills the entries itself and never touches a GPU)
      r->arena = static_cast<uint8_t*>(std::malloc(total));
      if (!r->arena) return fail(KVT_ERR_INVALID, "kvt_object_ring_create: out of memory");
    } else {
      if (int rc = check_device(device)) return rc;
      DeviceGuard g;
      if (int rc = g.enter(device)) return rc;
      KVT_HIP(hipHostMalloc(reinterpret_cast<void**>(&r->arena), total, hipHostMallocDefault));
      KVT_HIP(hipStreamCreateWithFlags(&r->copy, hipStreamNonBlocking));
      KVT_HIP(hipEventCreateWithFlags(&r->fence, hipEventDisableTiming));
      KVT_HIP(hipEventCreateWithFlags(&r->meta_free, hipEventDisableTiming));
      const size_t meta_bytes = 3 * sizeof(int64_t) * static_cast<size_t>(n_entries);
      KVT_HIP(hipMalloc(reinterpret_cast<void**>(&r->meta_dev), meta_bytes));
      KVT_HIP(hipHostMalloc(reinterpret_cast<void**>(&r->meta_host), meta_bytes, hipHostMallocDefault));
    }
    *out = r.release();
    return KVT_OK;
  });
}

void kvt_object_ring_destroy(kvt_object_ring* r) {
  if (!r) return;
  if (r->copy) {
    (void)hipStreamSynchronize(r->copy);
    (void)hipStreamDestroy(r->copy);
  }
  r->entries.clear();   // drops the transfer events
  if (r->fence) (void)hipEventDestroy(r->fence);
  if (r->meta_free) (void)hipEventDestroy(r->meta_free);
  if (r->meta_dev) {
    forget_device_spans();
    (void)hipFree(r->meta_dev);
  }
  if (r->meta_host) (void)hipHostFree(r->meta_host);
  if (r->arena) {
    if (r->device == KVT_DEVICE_NONE)
      std::free(r->arena);
    else
      (void)hipHostFree(r->arena);
  }
  delete r;
}

void* kvt_object_ring_entry(kvt_object_ring* r, uint32_t entry) {
  return (r && entry < r->n_entries) ? r->arena + static_cast<uint64_t>(entry) * r->entry_bytes
                                     : nullptr;
}

int kvt_object_ring_reserve(kvt_object_ring* r, const void* keys, uint32_t n, uint32_t* entries,
                            uint8_t* is_new) {
  return guarded([&]() -> int {
    if (!r || (n && (!keys || !entries || !is_new)))
      return fail(KVT_ERR_INVALID, "kvt_object_ring_reserve: null argument");
    std::lock_guard<std::mutex> lock(r->mu);
    const uint64_t call = ++r->calls;
    const char* k = static_cast<const char*>(keys);
    // first the keys that are here already: their entries must survive this call
    uint32_t fresh = 0;
    std::vector<std::string> ks(n);
    for (uint32_t i = 0; i < n; ++i) {
      ks[i].assign(k + static_cast<size_t>(i) * r->key_bytes, r->key_bytes);
      auto it = r->index.find(ks[i]);
      if (it != r->index.end()) {
        r->entries[it->second].touched = call;
      }
    }
    {
      std::unordered_map<std::string, int> seen;
      for (uint32_t i = 0; i < n; ++i)
        if (!r->index.count(ks[i]) && seen.emplace(ks[i], 1).second) ++fresh;
    }
    // entries that may be given away: not referred to by this call, and not claimed by a caller
    // who has yet to write them (another thread between its reserve and its save)
    uint32_t available = 0;
    for (const Entry& e : r->entries)
      if (e.touched != call && e.claims == 0) ++available;
    if (fresh > available)
      return fail(KVT_ERR_INVALID,
                  "kvt_object_ring_reserve: more new blocks than entries that may be given away "
                  "(entries this batch refers to and reservations not yet written stay)");
    for (uint32_t i = 0; i < n; ++i) {
      auto it = r->index.find(ks[i]);
      if (it != r->index.end()) {
        Entry& e = r->entries[it->second];
        entries[i] = it->second;
        // present and written: nothing to do. Reserved before but never written: the caller
        // is asked again, once per call (a key may be repeated inside a batch).
        is_new[i] = (!e.saved && e.flagged != call) ? 1 : 0;
        if (is_new[i]) {
          e.flagged = call;
          ++e.claims;
          ++r->stats.blocks_asked_for;
        } else {
          ++r->stats.blocks_already_here;
        }
        continue;
      }
      uint32_t idx = 0;
      for (;;) {   // the oldest entry that may be given away
        idx = static_cast<uint32_t>(r->handed_out++ % r->n_entries);
        if (r->entries[idx].touched != call && r->entries[idx].claims == 0) break;
      }
      Entry& e = r->entries[idx];
      if (int rc = wait_entry(e)) return rc;
      if (!e.key.empty()) {
        r->index.erase(e.key);
        ++r->stats.entries_given_away;
      }
      ++r->stats.blocks_asked_for;
      e.key = ks[i];
      e.saved = false;
      e.claims = 1;
      e.touched = call;
      e.flagged = call;
      r->index.emplace(ks[i], idx);
      entries[i] = idx;
      is_new[i] = 1;
    }
    return KVT_OK;
  });
}

int kvt_object_ring_lookup(kvt_object_ring* r, const void* keys, uint32_t n, uint32_t* entries,
                           uint8_t* found) {
  return guarded([&]() -> int {
    if (!r || (n && (!keys || !entries || !found)))
      return fail(KVT_ERR_INVALID, "kvt_object_ring_lookup: null argument");
    std::lock_guard<std::mutex> lock(r->mu);
    const char* k = static_cast<const char*>(keys);
    std::string key;
    for (uint32_t i = 0; i < n; ++i) {
      key.assign(k + static_cast<size_t>(i) * r->key_bytes, r->key_bytes);
      auto it = r->index.find(key);
      found[i] = (it != r->index.end() && r->entries[it->second].saved) ? 1 : 0;
      entries[i] = found[i] ? it->second : 0;
      ++(found[i] ? r->stats.lookups_found : r->stats.lookups_missed);
    }
    return KVT_OK;
  });
}

int kvt_object_ring_commit(kvt_object_ring* r, const uint32_t* entries, uint32_t n) {
  return guarded([&]() -> int {
    if (!r || (n && !entries)) return fail(KVT_ERR_INVALID, "kvt_object_ring_commit: null argument");
    std::lock_guard<std::mutex> lock(r->mu);
    if (int rc = check_entries(r, entries, n, "kvt_object_ring_commit")) return rc;
    for (uint32_t i = 0; i < n; ++i) {
      Entry& e = r->entries[entries[i]];
      e.saved = true;
      if (e.claims) --e.claims;
    }
    return KVT_OK;
  });
}

int kvt_object_ring_release(kvt_object_ring* r, const uint32_t* entries, uint32_t n) {
  return guarded([&]() -> int {
    if (!r || (n && !entries)) return fail(KVT_ERR_INVALID, "kvt_object_ring_release: null argument");
    std::lock_guard<std::mutex> lock(r->mu);
    for (uint32_t i = 0; i < n; ++i)
      if (entries[i] >= r->n_entries)
        return fail(KVT_ERR_OUT_OF_RANGE, "kvt_object_ring_release: entry index out of range");
    for (uint32_t i = 0; i < n; ++i) {
      Entry& e = r->entries[entries[i]];
      if (e.key.empty() || e.claims == 0) continue;   // nothing claimed here
      if (--e.claims == 0 && !e.saved) {              // nobody is going to write it: forget the key
        r->index.erase(e.key);
        e.key.clear();
      }
    }
    return KVT_OK;
  });
}

int kvt_object_ring_stats(kvt_object_ring* r, kvt_object_ring_counters* out) {
  if (!r || !out) return fail(KVT_ERR_INVALID, "kvt_object_ring_stats: null argument");
  std::lock_guard<std::mutex> lock(r->mu);
  *out = r->stats;
  out->entries_in_use = r->index.size();
  return KVT_OK;
}

int kvt_object_ring_wait(kvt_object_ring* r, uint32_t entry) {
  return guarded([&]() -> int {
    if (!r || entry >= r->n_entries) return fail(KVT_ERR_INVALID, "kvt_object_ring_wait: bad argument");
    std::shared_ptr<Transfer> t;
    {
      std::lock_guard<std::mutex> lock(r->mu);
      t = r->entries[entry].pending;
    }
    if (t) KVT_HIP(hipEventSynchronize(t->done));
    return KVT_OK;
  });
}

// save = true: device -> entries (and the entries count as written); false: entries -> device.
static int transfer(kvt_object_ring* r, const uint32_t* entries, uint32_t n, void* dev,
                    uint64_t dev_stride, void* stream, bool save, const void* keys = nullptr) {
  const char* who = save ? "kvt_object_ring_save" : "kvt_object_ring_load";
  if (!r || (n && (!entries || !dev))) return fail(KVT_ERR_INVALID, std::string(who) + ": null argument");
  if (n == 0) return KVT_OK;
  if (r->device == KVT_DEVICE_NONE)
    return fail(KVT_ERR_NO_DEVICE, std::string(who) + ": this ring was created without a device");
  if (dev_stride < r->entry_bytes)
    return fail(KVT_ERR_INVALID, std::string(who) + ": device stride smaller than an entry");
  std::lock_guard<std::mutex> lock(r->mu);
  if (int rc = check_entries(r, entries, n, who)) return rc;
  if (!save)
    for (uint32_t i = 0; i < n; ++i) {
      const Entry& e = r->entries[entries[i]];
      if (!e.saved) return fail(KVT_ERR_INVALID, "kvt_object_ring_load: entry has not been written");
      if (keys && std::memcmp(e.key.data(), static_cast<const char*>(keys) + static_cast<size_t>(i) * r->key_bytes,
                              r->key_bytes) != 0)
        return fail(KVT_ERR_OUT_OF_RANGE,
                    "kvt_object_ring_load: an entry was given to another block since the lookup");
    }
  DeviceGuard g;
  if (int rc = g.enter(r->device)) return rc;
  uint64_t extent = 0;
  if (__builtin_mul_overflow(static_cast<uint64_t>(n - 1), dev_stride, &extent) ||
      __builtin_add_overflow(extent, r->entry_bytes, &extent))
    return fail(KVT_ERR_OUT_OF_RANGE, std::string(who) + ": device stride times entries exceeds 64 bits");
  if (int rc = check_device_span(dev, extent, std::string(who) + ": the device buffer")) return rc;
  const hipStream_t user = static_cast<hipStream_t>(stream);
  // behind whatever the caller's stream has queued (the pack that produces the objects, or the
  // kernels still reading the buffer a load is about to overwrite)
  KVT_HIP(hipEventRecord(r->fence, user));
  KVT_HIP(hipStreamWaitEvent(r->copy, r->fence, 0));
  uint8_t* d = static_cast<uint8_t*>(dev);
  // Pieces: runs of entries that are neighbours on both sides. A few long ones go to the DMA
  // engines, one copy each; many short ones are moved by ONE launch of the range kernel,
  // which crosses PCIe at 56 GB/s whatever their length (a DMA copy of 2 MiB reaches 33).
  static thread_local std::vector<kvt_ipc_block> pieces;
  pieces.clear();
  (void)for_runs(r, entries, n, dev_stride, [&](uint32_t first, uint32_t count) -> int {
    pieces.push_back(kvt_ipc_block{static_cast<uint64_t>(entries[first]) * r->entry_bytes,
                                   static_cast<uint64_t>(first) * dev_stride,
                                   static_cast<uint64_t>(count) * r->entry_bytes});
    return KVT_OK;
  });
  const uint64_t moved = static_cast<uint64_t>(n) * r->entry_bytes;
  if (pieces.size() > 1 && moved / pieces.size() < (8ull << 20) && pieces.size() <= r->n_entries) {
    if (r->meta_used) KVT_HIP(hipEventSynchronize(r->meta_free));  // the staging area is free again
    const uint64_t m = pieces.size();
    if (int rc = kvt_copy_handle_data_kernel_direct(
            r->arena, d, pieces.data(), m, static_cast<uint64_t>(r->n_entries) * r->entry_bytes,
            save ? KVT_COPY_D2H : KVT_COPY_H2D, r->device, r->copy, r->meta_dev, r->meta_dev + m,
            r->meta_dev + 2 * m, r->meta_host, 1))
      return rc;
    KVT_HIP(hipEventRecord(r->meta_free, r->copy));
    r->meta_used = true;
  } else if (int rc = for_runs(r, entries, n, dev_stride, [&](uint32_t first, uint32_t count) -> int {
        uint8_t* host = r->arena + static_cast<uint64_t>(entries[first]) * r->entry_bytes;
        uint8_t* devp = d + static_cast<uint64_t>(first) * dev_stride;
        const uint64_t bytes = static_cast<uint64_t>(count) * r->entry_bytes;
        if (save)
          KVT_HIP(hipMemcpyAsync(host, devp, bytes, hipMemcpyDeviceToHost, r->copy));
        else
          KVT_HIP(hipMemcpyAsync(devp, host, bytes, hipMemcpyHostToDevice, r->copy));
        return KVT_OK;
      }))
    return rc;
  (save ? r->stats.bytes_saved : r->stats.bytes_loaded) += static_cast<uint64_t>(n) * r->entry_bytes;
  auto t = std::make_shared<Transfer>();
  KVT_HIP(hipEventCreateWithFlags(&t->done, hipEventDisableTiming));
  KVT_HIP(hipEventRecord(t->done, r->copy));
  for (uint32_t i = 0; i < n; ++i) {
    Entry& e = r->entries[entries[i]];
    e.pending = t;
    if (save) {
      e.saved = true;
      if (e.claims) --e.claims;
    }
  }
  // the caller's stream continues once the bytes have moved: a load is followed by the unpack
  // that reads them, a save by whatever reuses the device buffer
  KVT_HIP(hipStreamWaitEvent(user, t->done, 0));
  return KVT_OK;
}

int kvt_object_ring_save(kvt_object_ring* r, const uint32_t* entries, uint32_t n, const void* dev,
                         uint64_t dev_stride, void* stream) {
  return guarded([&]() -> int {
    return transfer(r, entries, n, const_cast<void*>(dev), dev_stride, stream, true);
  });
}

int kvt_object_ring_load(kvt_object_ring* r, const uint32_t* entries, const void* keys, uint32_t n,
                         void* dev, uint64_t dev_stride, void* stream) {
  return guarded([&]() -> int {
    return transfer(r, entries, n, dev, dev_stride, stream, false, keys);
  });
}

}  // extern "C"
