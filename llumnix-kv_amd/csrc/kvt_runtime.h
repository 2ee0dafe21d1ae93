// Internal declarations shared by the HIP translation units of libkvt_hip
// (device selection, the chunk-table pool, registered caches and copy plans).
#ifndef KVT_RUNTIME_H_
#define KVT_RUNTIME_H_

#include <hip/hip_runtime.h>

#include <atomic>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "kvt_device.h"
#include "kvt_internal.h"

namespace kvt {

int hip_fail(hipError_t e, const char* what);

#define KVT_HIP(call)                                  \
  do {                                                 \
    const hipError_t _e = (call);                      \
    if (_e != hipSuccess) return hip_fail(_e, #call);  \
  } while (0)

// Number of devices, or 0. Only gfx950 parts are accepted: the code objects in
// this library are built for that target alone.
int usable_devices();
// KVT_OK, or KVT_ERR_NO_DEVICE / KVT_ERR_INVALID with the message set.
int check_device(int device);

// The most workgroups one copy launch may use on `device`, or 0 for no limit
// (kvt_set_copy_cu_usage).
uint32_t copy_wg_cap(int device);
// Compute units of `device` (0 when unknown).
uint32_t device_cu_count(int device);

// KVT_OK when [ptr, ptr + bytes) is, as far as the runtime can tell, memory the device may
// touch; KVT_ERR_INVALID / KVT_ERR_OUT_OF_RANGE (message set, starting with `what`) otherwise.
// *host_memory (optional): the pointer is host memory mapped into the device (pinned), i.e.
// whatever a kernel moves there crosses PCIe.
int check_device_span(const void* ptr, uint64_t bytes, const std::string& what, bool* host_memory = nullptr);
// Launches whose payload is at most this many bytes read with plain loads (kvt_set_copy_cached_load_max).
uint64_t copy_cached_load_max_bytes();
// ... write with plain stores (kvt_set_copy_cached_store_max).
uint64_t copy_cached_store_max_bytes();
// Drops every remembered allocation extent (call where device memory is freed).
void forget_device_spans();

struct DeviceGuard {
  int prev = -1;
  bool switched = false;
  int enter(int device) {
    if (hipGetDevice(&prev) != hipSuccess) prev = -1;
    if (prev != device) {
      const hipError_t e = hipSetDevice(device);
      if (e != hipSuccess) return hip_fail(e, "hipSetDevice");
      switched = true;
    }
    return KVT_OK;
  }
  ~DeviceGuard() {
    if (switched && prev >= 0) (void)hipSetDevice(prev);
  }
};

inline uint64_t round_up(uint64_t v, uint64_t a) { return (v + a - 1) / a * a; }

// Ticket blocks of the persistent (CU-share limited) kernels: nine 32-bit counters, 128 bytes
// apart, from which the workgroups of ONE launch take their work (kvt_kernels.hip, EntryWalk).
// A block is all zero when a launch starts and the launch leaves it all zero, so the only rule
// is that two launches that may run at the same time never share one. An eager launch borrows
// a block until the event recorded behind it has completed; a launch recorded into a hipGraph
// keeps its block for as long as the plan's table lives (every replay uses it again). The
// blocks of a device are allocated in one piece when a CU share is first set for it -- never
// during a launch, which may sit inside a stream capture -- and a launch that finds none free
// runs without tickets (static striding), slower but as correct.
class TicketPool {
 public:
  static constexpr uint32_t kBlockBytes = 2048, kBlocks = 1024;
  // blocks [0, kEagerBlocks) are lent to eager launches, the rest belong to captured ones
  static constexpr uint32_t kEagerBlocks = 768;
  // Allocates the device's blocks (no-op when they exist). Not inside a stream capture.
  int prepare(int device);
  // A block no running launch uses, or nullptr. permanent (a launch that is being recorded
  // into a stream capture): taken out of circulation until give_back(), found without any
  // call into the runtime; otherwise the caller calls launched() once the kernel is on `stream`.
  uint32_t* acquire(int device, bool permanent);
  // {eager launches that got a block, eager launches that found none, captured launches that
  // got one, captured launches that found none} since the device's blocks were allocated.
  void stats(int device, uint64_t out[4]);
  void launched(int device, uint32_t* block, hipStream_t stream);
  // A permanent block whose graph is gone, or a borrowed one whose launch never happened.
  void give_back(int device, uint32_t* block);

 private:
  enum State : uint8_t { kFree = 0, kLent = 1, kInFlight = 2, kPermanent = 3 };  // kLent: event not recorded yet
  struct PerDevice {
    uint8_t* arena = nullptr;
    std::vector<hipEvent_t> done;
    std::vector<uint8_t> state;
    uint32_t cursor = 0, capture_cursor = 0;
    uint64_t counters[4] = {0, 0, 0, 0};
  };
  PerDevice* of(int device);  // under mu_
  std::mutex mu_;
  std::vector<PerDevice> devices_;
};
TicketPool& ticket_pool();

// Chunk tables are uploaded once per batch and die with the batch. hipMalloc /
// hipFree per batch would stall (hipFree waits for the whole device), so table
// storage is recycled: a buffer = device memory + a pinned host twin of the same
// size + one event per stream that has launched kernels reading it, marking the
// last such launch. A released buffer is handed out again only once all of them
// have completed.
struct TableBuf {
  struct Use {
    hipStream_t stream;
    hipEvent_t done;
    bool recorded;
  };
  int device = -1;
  size_t cap = 0;
  void* dev = nullptr;
  void* host = nullptr;   // pinned staging for the asynchronous upload
  std::mutex mu;          // a plan may be launched from several threads
  std::vector<Use> uses;  // events are kept across recycling (streams repeat)
  bool captured = false;  // read by a kernel recorded into a hipGraph
  std::vector<uint32_t*> graph_tickets;  // ticket blocks of launches recorded into a hipGraph (under mu)
  // which of them serves which capture: launches recorded into one capture on one stream share
  // a block (under mu)
  struct CaptureTickets {
    unsigned long long capture;
    hipStream_t stream;
    uint32_t* block;
  };
  std::vector<CaptureTickets> capture_tickets;

  // Call after every launch on `stream` that reads `dev`.
  int mark_use(hipStream_t stream) {
    std::lock_guard<std::mutex> lock(mu);
    Use* u = nullptr;
    for (Use& x : uses)
      if (x.stream == stream) u = &x;
    if (!u) {
      if (uses.size() >= 16) {  // many streams: retire the oldest entry instead of growing
        if (uses.front().recorded) KVT_HIP(hipEventSynchronize(uses.front().done));
        uses.front().recorded = false;
        uses.front().stream = stream;
        u = &uses.front();
      } else {
        hipEvent_t ev = nullptr;
        KVT_HIP(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
        uses.push_back(Use{stream, ev, false});
        u = &uses.back();
      }
    }
    KVT_HIP(hipEventRecord(u->done, stream));
    u->recorded = true;
    return KVT_OK;
  }
  // No queued kernel reads the table any more.
  bool idle() {
    std::lock_guard<std::mutex> lock(mu);
    for (const Use& x : uses)
      if (x.recorded && hipEventQuery(x.done) != hipSuccess) {
        (void)hipGetLastError();
        return false;
      }
    return true;
  }
  void wait_idle() {
    std::lock_guard<std::mutex> lock(mu);
    for (const Use& x : uses)
      if (x.recorded) (void)hipEventSynchronize(x.done);
  }
  void forget_uses() {
    std::lock_guard<std::mutex> lock(mu);
    for (Use& x : uses) x.recorded = false;
  }
};

class TablePool {
 public:
  int acquire(int device, size_t bytes, TableBuf** out) {
    {
      std::lock_guard<std::mutex> lock(mu_);
      size_t best = idle_.size();
      for (size_t i = 0; i < idle_.size(); ++i) {
        TableBuf* b = idle_[i];
        if (b->device != device || b->cap < bytes) continue;
        if (!b->idle()) continue;  // still being read by a queued kernel
        if (best == idle_.size() || b->cap < idle_[best]->cap) best = i;
      }
      if (best != idle_.size()) {
        *out = idle_[best];
        idle_bytes_ -= idle_[best]->cap;
        idle_.erase(idle_.begin() + best);
        (*out)->forget_uses();
        return KVT_OK;
      }
    }
    std::unique_ptr<TableBuf> b(new TableBuf());
    b->device = device;
    b->cap = 65536;
    while (b->cap < bytes) b->cap *= 2;
    KVT_HIP(hipMalloc(&b->dev, b->cap));
    const hipError_t e = hipHostMalloc(&b->host, b->cap, hipHostMallocDefault);
    if (e != hipSuccess) {
      destroy(b.get());
      return hip_fail(e, "table buffer allocation");
    }
    *out = b.release();
    return KVT_OK;
  }

  void release(TableBuf* b) {
    if (!b) return;
    if (b->captured) {  // a graph may replay the kernel later: never recycle, free for good
      destroy(b);
      delete b;
      return;
    }
    std::vector<TableBuf*> victims;
    {
      std::lock_guard<std::mutex> lock(mu_);
      idle_.push_back(b);
      idle_bytes_ += b->cap;
      // Freeing device memory waits for the whole device, so a serving loop must not get
      // here: the pool is bounded by the memory it holds (tables are 64 KiB to a few MiB; the
      // bound is hundreds of batches), not by a count that a burst of small plans reaches.
      // Over the bound it shrinks to three quarters at once, oldest first.
      if (idle_bytes_ > kMaxIdleBytes || idle_.size() > kMaxIdle) {
        size_t n = 0;
        while (n + 1 < idle_.size() &&
               (idle_bytes_ > kMaxIdleBytes / 4 * 3 || idle_.size() - n > kMaxIdle / 4 * 3)) {
          idle_bytes_ -= idle_[n]->cap;
          ++n;
        }
        victims.assign(idle_.begin(), idle_.begin() + n);
        idle_.erase(idle_.begin(), idle_.begin() + n);
      }
    }
    for (TableBuf* victim : victims) {
      victim->wait_idle();
      destroy(victim);
      delete victim;
    }
  }

  // One upload stream per device, created on first use.
  int upload_stream(int device, hipStream_t* out) {
    std::lock_guard<std::mutex> lock(mu_);
    if (device >= static_cast<int>(streams_.size())) streams_.resize(device + 1, nullptr);
    if (!streams_[device]) KVT_HIP(hipStreamCreateWithFlags(&streams_[device], hipStreamNonBlocking));
    *out = streams_[device];
    return KVT_OK;
  }

 private:
  static constexpr size_t kMaxIdle = 4096;
  static constexpr size_t kMaxIdleBytes = size_t(256) << 20;  // device memory, and as much pinned
 public:
  // Frees what a buffer holds (device memory, pinned twin, events; its graphs' ticket blocks go
  // back to their pool).
  static void destroy(TableBuf* b) {
    for (uint32_t* t : b->graph_tickets) ticket_pool().give_back(b->device, t);
    b->graph_tickets.clear();
    b->capture_tickets.clear();
    if (b->dev) (void)hipFree(b->dev);
    if (b->host) (void)hipHostFree(b->host);
    for (TableBuf::Use& u : b->uses) (void)hipEventDestroy(u.done);
    b->uses.clear();
    b->dev = b->host = nullptr;
  }

 private:
  std::mutex mu_;
  std::vector<TableBuf*> idle_;
  size_t idle_bytes_ = 0;
  std::vector<hipStream_t> streams_;
};

TablePool& table_pool();

constexpr uint32_t kMinChunk = 4096, kMaxAutoChunk = 32768, kMaxChunk = 1u << 19;
constexpr uint64_t kBlobAlign = 256;

}  // namespace kvt

struct kvt_cache {
  int device = 0;
  uint32_t n_layers = 0, n_tensors = 0;
  std::vector<uint64_t> capacity;
  std::vector<void*> host_ptrs;
  uint8_t** dev_ptrs = nullptr;
  bool aligned16 = true;  // every layer tensor starts on a 16-byte boundary
  bool aligned4 = true;   // ... on a 4-byte boundary
};

namespace kvt {
// A plan slot (kvt_plan_slot_create): the plan's table lives at a fixed device address with a
// header in front (SlotHeader) and is rewritten for every batch by kvt_plan_slot_fill, through
// one of two pinned staging copies in turn. The plan's TableBuf holds the device memory (never
// recycled through the pool) and the record of eager launches that still read it.
struct Slot {
  int kind = kSlotPlain;
  uint64_t max_entries = 0, max_layer_bytes = 0;
  uint32_t chunk_bytes = 0;
  uint32_t ntpb = 0;                 // layout transform: tokens per page
  uint64_t half = 0, tok_bytes = 0;  // ... bytes of a half page and of one token row
  uint8_t* host[2] = {nullptr, nullptr};
  hipEvent_t staged[2] = {nullptr, nullptr};  // the copy out of host[i] has run
  bool staged_rec[2] = {false, false};
  uint32_t turn = 0;
  hipEvent_t filled = nullptr;       // the newest contents have reached the device
  hipStream_t filled_on = nullptr;
  bool filled_rec = false;
  std::mutex mu;                     // a fill against launches from other threads
};
}  // namespace kvt

struct kvt_plan {
  int device = 0;
  kvt::Slot* slot = nullptr;       // non-null: a plan slot, refilled per batch
  uint32_t n_tensors = 0;
  uint64_t n_chunks = 0;
  std::vector<uint64_t> tensor_bytes, tensor_offset, src_cap, dst_cap;
  uint64_t layer_bytes = 0;
  uint64_t min_layer_stride = 0;   // smallest layer_stride a multi-layer launch accepts
  bool xform = false;
  kvt::XformDev xdev{};
  bool strided = false;            // some chunks carry a record shape (kvt_plan_create_runs)
  kvt::StrideTable shapes{};
  uint64_t n_strided = 0;
  bool convert = false;            // pack converts bf16 -> fp8: lengths count fp8 bytes (elements)
  bool all16 = false;              // every entry's offsets and length are multiples of 16 bytes
  bool near = true;                // no entry spans 2 GiB or more on the cache side (32-bit offsets do)
  std::vector<kvt::Chunk> host_table;   // device == KVT_DEVICE_NONE only: the tables, kept on the host
  uint32_t sub_shift = 0;          // chunks hold at most 4096 << sub_shift bytes
  // plain plans of at most kSmallTable entries: both tables kept here and passed to the
  // kernel by value; no device table, no upload
  bool small = false;
  kvt::SmallTable small_pack{}, small_unpack{};
  kvt::Chunk* dev_chunks = nullptr;     // [0, n_chunks): pack order; [n_chunks, 2 n_chunks): unpack order
  kvt::TableBuf* buf = nullptr;         // storage of dev_chunks (recycled through the table pool)
  hipEvent_t uploaded = nullptr;   // completes when the table has reached the device
  // a launch has already observed `uploaded` as complete (several threads may launch one plan)
  mutable std::atomic<bool> upload_seen{false};
};

namespace kvt {

// Launches the pack (gather) or unpack (scatter) of layers [first_layer, first_layer +
// n_layers) of a plan. blob_offsets = nullptr: the plan's own blob positions.
int run_plan(bool pack, const kvt_plan* p, const kvt_cache* cache, uint32_t first_layer,
             uint32_t n_layers, void* packed, uint64_t layer_stride, void* stream,
             const uint64_t* blob_offsets = nullptr);

}  // namespace kvt

#endif  // KVT_RUNTIME_H_
