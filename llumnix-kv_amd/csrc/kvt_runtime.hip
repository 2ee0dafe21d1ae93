// Host side of the device path: registered caches, copy plans, pack / unpack
// launches, the reference-shaped copy entry points, per-layer gating sessions
// and pinned-host staging.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <condition_variable>
#include <cstring>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "kvt_device.h"
#include "kvt_internal.h"

namespace kvt {
namespace {

int hip_fail(hipError_t e, const char* what) {
  return fail(KVT_ERR_HIP, std::string(what) + ": " + hipGetErrorString(e));
}

#define KVT_HIP(call)                                  \
  do {                                                 \
    const hipError_t _e = (call);                      \
    if (_e != hipSuccess) return hip_fail(_e, #call);  \
  } while (0)

// Number of devices, or a negative KVT error. Only gfx950 parts are accepted:
// the code objects in this library are built for that target alone.
int usable_devices() {
  static int cached = -2;
  static std::once_flag once;
  std::call_once(once, []() {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
      (void)hipGetLastError();
      cached = 0;
      return;
    }
    int ok = 0;
    for (int i = 0; i < n; ++i) {
      hipDeviceProp_t p;
      if (hipGetDeviceProperties(&p, i) != hipSuccess) break;
      if (std::strncmp(p.gcnArchName, "gfx950", 6) != 0) break;
      ++ok;
    }
    cached = ok;
  });
  return cached;
}

int check_device(int device) {
  const int n = usable_devices();
  if (n <= 0) return fail(KVT_ERR_NO_DEVICE, "no usable gfx950 (MI355X) device");
  if (device < 0 || device >= n) return fail(KVT_ERR_INVALID, "device index out of range");
  return KVT_OK;
}

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

uint64_t round_up(uint64_t v, uint64_t a) { return (v + a - 1) / a * a; }

// Chunk tables are uploaded once per batch and die with the batch. hipMalloc /
// hipFree per batch would stall (hipFree waits for the whole device), so table
// storage is recycled: a buffer = device memory + a pinned host twin of the same
// size + an event that marks its last use on the GPU. A released buffer is handed
// out again only once that event has completed.
struct TableBuf {
  int device = -1;
  size_t cap = 0;
  void* dev = nullptr;
  void* host = nullptr;          // pinned staging for the asynchronous upload
  hipEvent_t last_use = nullptr; // recorded after every launch that reads `dev`
  bool used = false;             // last_use has been recorded at least once
  bool captured = false;         // read by a kernel recorded into a hipGraph
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
        if (b->used && hipEventQuery(b->last_use) != hipSuccess) {
          (void)hipGetLastError();
          continue;  // still being read by a queued kernel
        }
        if (best == idle_.size() || b->cap < idle_[best]->cap) best = i;
      }
      if (best != idle_.size()) {
        *out = idle_[best];
        idle_.erase(idle_.begin() + best);
        (*out)->used = false;
        return KVT_OK;
      }
    }
    std::unique_ptr<TableBuf> b(new TableBuf());
    b->device = device;
    b->cap = 65536;
    while (b->cap < bytes) b->cap *= 2;
    KVT_HIP(hipMalloc(&b->dev, b->cap));
    hipError_t e = hipHostMalloc(&b->host, b->cap, hipHostMallocDefault);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&b->last_use, hipEventDisableTiming);
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
    std::lock_guard<std::mutex> lock(mu_);
    if (idle_.size() >= 64) {
      TableBuf* victim = idle_.front();
      idle_.erase(idle_.begin());
      if (victim->used) (void)hipEventSynchronize(victim->last_use);
      destroy(victim);
      delete victim;
    }
    idle_.push_back(b);
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
  static void destroy(TableBuf* b) {
    if (b->dev) (void)hipFree(b->dev);
    if (b->host) (void)hipHostFree(b->host);
    if (b->last_use) (void)hipEventDestroy(b->last_use);
    b->dev = b->host = nullptr;
    b->last_use = nullptr;
  }
  std::mutex mu_;
  std::vector<TableBuf*> idle_;
  std::vector<hipStream_t> streams_;
};

TablePool& table_pool() {
  static TablePool* pool = new TablePool();  // intentionally leaked: outlives static destruction
  return *pool;
}

constexpr uint32_t kMinChunk = 4096, kMaxAutoChunk = 32768, kMaxChunk = 1u << 19;
constexpr uint64_t kBlobAlign = 256;


// One table entry before sorting.
struct Piece {
  uint64_t src, dst, packed;
  uint32_t len;
  uint16_t tensor, t0;
  uint32_t shape;
};

// Every table entry is served by chunk_bytes / 4096 workgroups, of which only
// ceil(len / 4096) have bytes to move. Takes the largest entry size (fewest table
// entries) that leaves at most 2 % of the launched workgroups idle. `spans` holds
// (bytes, repetitions) of the contiguous-on-the-packed-side spans to be cut.
uint32_t pick_chunk_bytes(const std::vector<std::pair<uint64_t, uint64_t>>& spans) {
  for (uint32_t cand = kMaxAutoChunk; cand > kMinChunk; cand /= 2) {
    uint64_t launched = 0, useful = 0;
    for (const auto& sp : spans) {
      launched += sp.second * ((sp.first + cand - 1) / cand) * (cand / kMinChunk);
      useful += sp.second * ((sp.first + kMinChunk - 1) / kMinChunk);
    }
    if (launched * 100 <= useful * 102) return cand;
  }
  return kMinChunk;
}

}  // namespace
}  // namespace kvt

using namespace kvt;

struct kvt_cache {
  int device = 0;
  uint32_t n_layers = 0, n_tensors = 0;
  std::vector<uint64_t> capacity;
  std::vector<void*> host_ptrs;
  uint8_t** dev_ptrs = nullptr;
  bool aligned16 = true;  // every layer tensor starts on a 16-byte boundary
};

struct kvt_plan {
  int device = 0;
  uint32_t n_tensors = 0;
  uint64_t n_chunks = 0;
  std::vector<uint64_t> tensor_bytes, tensor_offset, src_cap, dst_cap;
  uint64_t layer_bytes = 0;
  bool xform = false;
  XformDev xdev{};
  bool strided = false;            // some chunks carry a record shape (kvt_plan_create_runs)
  StrideTable shapes{};
  uint64_t n_strided = 0;
  std::vector<Chunk> host_table;   // device == KVT_DEVICE_NONE only: the tables, kept on the host
  uint32_t sub_shift = 0;          // chunks hold at most 4096 << sub_shift bytes
  Chunk* dev_chunks = nullptr;     // [0, n_chunks): pack order; [n_chunks, 2 n_chunks): unpack order
  TableBuf* buf = nullptr;         // storage of dev_chunks (recycled through the table pool)
  hipEvent_t uploaded = nullptr;   // completes when the table has reached the device
  mutable bool upload_seen = false;  // a launch has already observed `uploaded` as complete
};

struct kvt_session {
  const kvt_plan* plan = nullptr;
  const kvt_cache* cache = nullptr;
  void* packed = nullptr;
  uint64_t layer_stride = 0;
  hipStream_t side = nullptr;
  std::vector<hipEvent_t> ready, done;
  hipEvent_t last_done = nullptr;
  // which layers' packs have been issued (wait_layer may be called, from another thread,
  // before the forward pass reaches the layer)
  std::mutex mu;
  std::condition_variable issued_cv;
  std::vector<uint8_t> issued;
};

struct kvt_stager {
  int device = 0;
  uint64_t slot_bytes = 0;
  uint32_t n_slots = 0;
  uint8_t* pinned = nullptr;
  hipStream_t copy = nullptr;
  std::vector<hipEvent_t> slot_done;
  hipEvent_t fence = nullptr;
};

// Sorts the pieces into the two tables and starts their upload.
static int finish_plan(kvt_plan* p, const std::vector<Piece>& pieces) {
  p->n_chunks = pieces.size();
  if ((p->n_chunks << p->sub_shift) > 0x7FFFFFF0ull)
    return fail(KVT_ERR_INVALID, "kvt_plan_create: too many chunks for one launch");

  // Two tables. What matters most to HBM throughput is that the WRITES of a launch
  // ascend: the unpack table is sorted by destination offset (tensor-major: different
  // tensors are different allocations); the pack table keeps generation order, which is
  // ascending packed offset (for a merged list that is ascending source offset as well).
  // Measured on MI355X: pack of an unmerged batch 5.88 -> 6.27 TB/s against sorting the
  // pack table by source offset; unpack +6 % against leaving it unsorted.
  auto fill = [](Chunk& c, const Piece& q, uint64_t cache) {
    c.cache = cache;
    c.packed = q.packed;
    c.len = q.len;
    c.tensor = q.tensor;
    c.t0 = q.t0;
    c.shape = q.shape;
    c.reserved = 0;
  };
  static thread_local std::vector<uint32_t> order;
  static thread_local std::vector<uint64_t> keys;
  const size_t n = pieces.size();
  keys.resize(n);
  for (size_t i = 0; i < n; ++i) {
    if ((pieces[i].src | pieces[i].dst) >> 56)
      return fail(KVT_ERR_INVALID, "kvt_plan_create: offset beyond 2^56");
    keys[i] = (static_cast<uint64_t>(pieces[i].tensor) << 56) | pieces[i].dst;
  }
  stable_order_by_key(keys, order);
  auto build = [&](Chunk* table) {
    for (size_t i = 0; i < n; ++i) fill(table[i], pieces[i], pieces[i].src);
    for (size_t i = 0; i < n; ++i) fill(table[n + i], pieces[order[i]], pieces[order[i]].dst);
  };

  if (p->device == KVT_DEVICE_NONE) {
    p->host_table.resize(2 * n);
    build(p->host_table.data());
    return KVT_OK;
  }
  DeviceGuard g;
  if (int rc = g.enter(p->device)) return rc;
  if (n != 0) {
    // Asynchronous upload: the tables are written straight into the pinned twin and copied
    // on the library's upload stream; the first launch that uses the plan waits for
    // `uploaded` on its own stream.
    const size_t bytes = 2 * n * sizeof(Chunk);
    if (int rc = table_pool().acquire(p->device, bytes, &p->buf)) return rc;
    build(static_cast<Chunk*>(p->buf->host));
    p->dev_chunks = static_cast<Chunk*>(p->buf->dev);
    hipStream_t up = nullptr;
    if (int rc = table_pool().upload_stream(p->device, &up)) {
      table_pool().release(p->buf);
      p->buf = nullptr;
      return rc;
    }
    hipError_t e = hipEventCreateWithFlags(&p->uploaded, hipEventDisableTiming);
    if (e == hipSuccess) e = hipMemcpyAsync(p->buf->dev, p->buf->host, bytes, hipMemcpyHostToDevice, up);
    if (e == hipSuccess) e = hipEventRecord(p->uploaded, up);
    if (e != hipSuccess) {
      (void)hipStreamSynchronize(up);
      if (p->uploaded) (void)hipEventDestroy(p->uploaded);
      p->uploaded = nullptr;
      table_pool().release(p->buf);
      p->buf = nullptr;
      return hip_fail(e, "chunk table upload");
    }
  }
  return KVT_OK;
}

extern "C" {

int kvt_device_count(void) { return std::max(0, usable_devices()); }

// ------------------------------------------------------------------- cache

int kvt_cache_register(int device, const void* const* ptrs, uint32_t n_layers, uint32_t n_tensors,
                       const uint64_t* capacity, kvt_cache** out) {
  return guarded([&]() -> int {
    if (!ptrs || !capacity || !out || n_layers == 0 || n_tensors == 0)
      return fail(KVT_ERR_INVALID, "kvt_cache_register: bad argument");
    if (n_tensors > KVT_MAX_TENSORS)
      return fail(KVT_ERR_INVALID, "kvt_cache_register: too many tensors per layer");
    if (int rc = check_device(device)) return rc;
    const uint64_t n = static_cast<uint64_t>(n_layers) * n_tensors;
    for (uint64_t i = 0; i < n; ++i)
      if (!ptrs[i]) return fail(KVT_ERR_INVALID, "kvt_cache_register: null layer pointer");
    DeviceGuard g;
    if (int rc = g.enter(device)) return rc;
    std::unique_ptr<kvt_cache> c(new kvt_cache());
    c->device = device;
    c->n_layers = n_layers;
    c->n_tensors = n_tensors;
    c->capacity.assign(capacity, capacity + n_tensors);
    c->host_ptrs.resize(n);
    for (uint64_t i = 0; i < n; ++i) {
      c->host_ptrs[i] = const_cast<void*>(ptrs[i]);
      if (reinterpret_cast<uintptr_t>(ptrs[i]) & 15u) c->aligned16 = false;
    }
    KVT_HIP(hipMalloc(reinterpret_cast<void**>(&c->dev_ptrs), n * sizeof(void*)));
    const hipError_t e =
        hipMemcpy(c->dev_ptrs, c->host_ptrs.data(), n * sizeof(void*), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
      (void)hipFree(c->dev_ptrs);
      return hip_fail(e, "hipMemcpy(layer pointer table)");
    }
    *out = c.release();
    return KVT_OK;
  });
}

void kvt_cache_destroy(kvt_cache* c) {
  if (!c) return;
  if (c->dev_ptrs) (void)hipFree(c->dev_ptrs);
  delete c;
}

// -------------------------------------------------------------------- plan

int kvt_plan_create(int device, const kvt_block_lists* lists, const uint64_t* src_capacity,
                    const uint64_t* dst_capacity, const kvt_xform* xform, uint32_t chunk_bytes,
                    kvt_plan** out) {
  return guarded([&]() -> int {
    if (!lists || !src_capacity || !dst_capacity || !out)
      return fail(KVT_ERR_INVALID, "kvt_plan_create: null argument");
    if (lists->tensors.empty() || lists->tensors.size() > KVT_MAX_TENSORS)
      return fail(KVT_ERR_INVALID, "kvt_plan_create: tensor count out of range");
    if (device != KVT_DEVICE_NONE)
      if (int rc = check_device(device)) return rc;
    if (chunk_bytes != 0 && (chunk_bytes < kMinChunk || chunk_bytes > kMaxChunk ||
                             (chunk_bytes & (chunk_bytes - 1)) != 0))
      return fail(KVT_ERR_INVALID,
                  "kvt_plan_create: chunk_bytes must be a power of two in [4096, 524288]");

    std::unique_ptr<kvt_plan> p(new kvt_plan());
    p->device = device;
    p->n_tensors = static_cast<uint32_t>(lists->tensors.size());
    p->src_cap.assign(src_capacity, src_capacity + p->n_tensors);
    p->dst_cap.assign(dst_capacity, dst_capacity + p->n_tensors);

    uint64_t half = 0, tok_bytes = 0;
    if (xform && xform->kind != KVT_XFORM_NONE) {
      if (xform->kind != KVT_XFORM_HND_NHD) return fail(KVT_ERR_INVALID, "unknown layout transform");
      if (p->n_tensors != 1) return fail(KVT_ERR_INVALID, "layout transform needs a single tensor");
      if (xform->heads == 0 || xform->ntpb == 0 || xform->row_bytes == 0 ||
          xform->row_bytes % 16 != 0 || xform->ntpb > 65535 || xform->heads > 65535)
        return fail(KVT_ERR_INVALID, "layout transform: rows must be multiples of 16 bytes");
      tok_bytes = static_cast<uint64_t>(xform->heads) * xform->row_bytes;
      half = tok_bytes * xform->ntpb;
      if (tok_bytes > kMaxChunk) return fail(KVT_ERR_INVALID, "layout transform: token row too large");
      p->xform = true;
      p->xdev.heads = xform->heads;
      p->xdev.ntpb = xform->ntpb;
      p->xdev.vrow = xform->row_bytes / 16;
      p->xdev.inv_vrow = static_cast<uint32_t>((1ull << 32) / p->xdev.vrow) + 1u;
      p->xdev.inv_heads = static_cast<uint32_t>((1ull << 32) / p->xdev.heads) + 1u;
    }

    if (chunk_bytes == 0) {
      std::vector<std::pair<uint64_t, uint64_t>> spans;
      for (const RunList& runs : lists->tensors)
        for (const kvt_ipc_block& r : runs)
          spans.emplace_back(p->xform ? half : r.length,
                             p->xform ? r.length / std::max<uint64_t>(half, 1) : 1);
      chunk_bytes = pick_chunk_bytes(spans);
    }
    if (p->xform)  // a chunk holds whole tokens
      while (chunk_bytes < tok_bytes) chunk_bytes *= 2;
    while ((kMinChunk << p->sub_shift) < chunk_bytes) ++p->sub_shift;

    // scratch kept per thread: a plan is built per batch, fresh pages every time would cost
    // more than filling them
    static thread_local std::vector<Piece> pieces;
    pieces.clear();
    uint64_t cursor = 0;
    for (uint32_t t = 0; t < p->n_tensors; ++t) {
      cursor = round_up(cursor, kBlobAlign);
      p->tensor_offset.push_back(cursor);
      uint64_t bad = 0;
      const RunList& runs = lists->tensors[t];
      if (kvt_validate_ipc_block_bounds(runs.data(), runs.size(), p->src_cap[t], 0, 1, &bad) ||
          kvt_validate_ipc_block_bounds(runs.data(), runs.size(), p->dst_cap[t], 1, 1, &bad))
        return fail(KVT_ERR_OUT_OF_RANGE, "kvt_plan_create: range " + std::to_string(bad) +
                                              " of tensor " + std::to_string(t) +
                                              " exceeds the stated capacity");
      uint64_t blob = 0;
      for (const kvt_ipc_block& r : runs) {
        if (!p->xform) {
          for (uint64_t o = 0; o < r.length; o += chunk_bytes)
            pieces.push_back(Piece{r.src_offset + o, r.dst_offset + o, blob + o,
                                   static_cast<uint32_t>(std::min<uint64_t>(chunk_bytes, r.length - o)),
                                   static_cast<uint16_t>(t), 0, 0});
        } else {
          const uint64_t page = 2 * half;
          if (r.src_offset % page || r.dst_offset % page || r.length % page)
            return fail(KVT_ERR_INVALID, "layout transform: ranges must be whole pages");
          const uint32_t tok_per_chunk = static_cast<uint32_t>(chunk_bytes / tok_bytes);
          for (uint64_t o = 0; o < r.length; o += half)  // one K or V half page at a time
            for (uint32_t t0 = 0; t0 < xform->ntpb; t0 += tok_per_chunk) {
              const uint32_t nt = std::min(tok_per_chunk, xform->ntpb - t0);
              pieces.push_back(Piece{r.src_offset + o, r.dst_offset + o,
                                     blob + o + static_cast<uint64_t>(t0) * tok_bytes,
                                     static_cast<uint32_t>(nt * tok_bytes), 0,
                                     static_cast<uint16_t>(t0), 0});
            }
        }
        blob += r.length;
      }
      p->tensor_bytes.push_back(blob);
      cursor += blob;
    }
    p->layer_bytes = round_up(cursor, kBlobAlign);
    if (int rc = finish_plan(p.get(), pieces)) return rc;
    *out = p.release();
    return KVT_OK;
  });
}

int kvt_plan_create_runs(int device, const kvt_run_lists* lists, const uint64_t* src_capacity,
                         const uint64_t* dst_capacity, uint32_t chunk_bytes, kvt_plan** out) {
  return guarded([&]() -> int {
    if (!lists || !src_capacity || !dst_capacity || !out)
      return fail(KVT_ERR_INVALID, "kvt_plan_create_runs: null argument");
    if (lists->tensors.empty() || lists->tensors.size() > KVT_MAX_TENSORS)
      return fail(KVT_ERR_INVALID, "kvt_plan_create_runs: tensor count out of range");
    if (device != KVT_DEVICE_NONE)
      if (int rc = check_device(device)) return rc;
    if (chunk_bytes != 0 && (chunk_bytes < kMinChunk || chunk_bytes > kMaxChunk ||
                             (chunk_bytes & (chunk_bytes - 1)) != 0))
      return fail(KVT_ERR_INVALID,
                  "kvt_plan_create_runs: chunk_bytes must be a power of two in [4096, 524288]");

    std::unique_ptr<kvt_plan> p(new kvt_plan());
    p->device = device;
    p->n_tensors = static_cast<uint32_t>(lists->tensors.size());
    p->src_cap.assign(src_capacity, src_capacity + p->n_tensors);
    p->dst_cap.assign(dst_capacity, dst_capacity + p->n_tensors);

    // A span is contiguous on the packed side: either one plain range, or the
    // records of one outermost iteration of a run that stays strided.
    struct Span {
      uint64_t src, dst, packed, bytes;
      uint32_t group;  // strided: bytes of one outer step (cut only there); 0 = plain
      uint32_t shape;
      uint64_t s_outer, d_outer;
      uint16_t tensor;
    };
    std::vector<Span> spans;
    uint32_t n_shapes = 0, max_group = 0;
    uint64_t cursor = 0;
    for (uint32_t t = 0; t < p->n_tensors; ++t) {
      cursor = round_up(cursor, kBlobAlign);
      p->tensor_offset.push_back(cursor);
      uint64_t blob = 0;
      const std::vector<kvt_run>& runs = lists->tensors[t];
      for (size_t ri = 0; ri < runs.size(); ++ri) {
        const kvt_run& r = runs[ri];
        // bounds: offsets grow with every index, so the last range decides
        uint64_t s_max = r.src_offset, d_max = r.dst_offset, count = 1;
        bool bad = r.length == 0 || r.n[0] == 0 || r.n[1] == 0 || r.n[2] == 0;
        for (int k = 0; k < 3 && !bad; ++k) {
          uint64_t ds, dd;
          bad = __builtin_mul_overflow(static_cast<uint64_t>(r.n[k] - 1), r.src_stride[k], &ds) ||
                __builtin_add_overflow(s_max, ds, &s_max) ||
                __builtin_mul_overflow(static_cast<uint64_t>(r.n[k] - 1), r.dst_stride[k], &dd) ||
                __builtin_add_overflow(d_max, dd, &d_max) ||
                __builtin_mul_overflow(count, static_cast<uint64_t>(r.n[k]), &count);
        }
        uint64_t total = 0;
        bad = bad || __builtin_mul_overflow(count, r.length, &total) ||
              s_max > p->src_cap[t] || r.length > p->src_cap[t] - s_max ||
              d_max > p->dst_cap[t] || r.length > p->dst_cap[t] - d_max;
        if (bad)
          return fail(KVT_ERR_OUT_OF_RANGE, "kvt_plan_create_runs: run " + std::to_string(ri) +
                                                " of tensor " + std::to_string(t) +
                                                " exceeds the stated capacity");
        // effective levels (n > 1), outermost first
        int lv[3], n_lv = 0;
        for (int k = 0; k < 3; ++k)
          if (r.n[k] > 1) lv[n_lv++] = k;
        bool strided = n_lv > 0 && r.length < kMinChunk && ((r.length | r.src_offset | r.dst_offset | blob) & 15u) == 0;
        for (int k = 0; k < n_lv && strided; ++k)
          strided = ((r.src_stride[lv[k]] | r.dst_stride[lv[k]]) & 15u) == 0;
        // kernel nest: (outer, inner) = the last two effective levels; an earlier one is cut here
        const int in_k = n_lv >= 2 ? lv[n_lv - 1] : -1;
        const int out_k = n_lv >= 2 ? lv[n_lv - 2] : (n_lv == 1 ? lv[0] : -1);
        const int top_k = n_lv == 3 ? lv[0] : -1;
        const uint64_t n_in = in_k >= 0 ? r.n[in_k] : 1;
        strided = strided && n_in * r.length <= kMaxChunk / 2;
        uint32_t shape = 0;
        if (strided) {
          StrideShape sh{};
          sh.vlen = static_cast<uint32_t>(r.length >> 4);
          sh.inv_vlen = static_cast<uint32_t>((1ull << 32) / sh.vlen) + 1u;
          sh.n_inner = static_cast<uint32_t>(n_in);
          sh.outer[0] = r.src_stride[out_k];
          sh.outer[1] = r.dst_stride[out_k];
          sh.inner[0] = in_k >= 0 ? r.src_stride[in_k] : 0;
          sh.inner[1] = in_k >= 0 ? r.dst_stride[in_k] : 0;
          for (uint32_t i = 0; i < n_shapes && !shape; ++i)
            if (std::memcmp(&p->shapes.shape[i], &sh, sizeof(sh)) == 0) shape = i + 1;
          if (!shape && n_shapes < kMaxShapes) {
            p->shapes.shape[n_shapes] = sh;
            shape = ++n_shapes;
          }
          strided = shape != 0;  // shape table full: expand this run
        }
        if (strided) {
          const uint32_t group = static_cast<uint32_t>(n_in * r.length);
          max_group = std::max(max_group, group);
          const uint64_t sub_bytes = static_cast<uint64_t>(r.n[out_k]) * group;
          const uint32_t n_top = top_k >= 0 ? r.n[top_k] : 1;
          for (uint32_t a = 0; a < n_top; ++a) {
            spans.push_back(Span{r.src_offset + (top_k >= 0 ? a * r.src_stride[top_k] : 0),
                                 r.dst_offset + (top_k >= 0 ? a * r.dst_stride[top_k] : 0), blob,
                                 sub_bytes, group, shape, r.src_stride[out_k], r.dst_stride[out_k],
                                 static_cast<uint16_t>(t)});
            blob += sub_bytes;
          }
        } else {
          for (uint32_t a = 0; a < r.n[0]; ++a)
            for (uint32_t b = 0; b < r.n[1]; ++b)
              for (uint32_t c = 0; c < r.n[2]; ++c) {
                spans.push_back(Span{
                    r.src_offset + a * r.src_stride[0] + b * r.src_stride[1] + c * r.src_stride[2],
                    r.dst_offset + a * r.dst_stride[0] + b * r.dst_stride[1] + c * r.dst_stride[2],
                    blob, r.length, 0, 0, 0, 0, static_cast<uint16_t>(t)});
                blob += r.length;
              }
        }
      }
      p->tensor_bytes.push_back(blob);
      cursor += blob;
    }
    p->layer_bytes = round_up(cursor, kBlobAlign);
    p->strided = n_shapes > 0;

    if (chunk_bytes == 0) {
      std::vector<std::pair<uint64_t, uint64_t>> sized;
      sized.reserve(spans.size());
      for (const Span& sp : spans) sized.emplace_back(sp.bytes, 1);
      chunk_bytes = pick_chunk_bytes(sized);
    }
    while (chunk_bytes < max_group) chunk_bytes *= 2;  // a chunk holds whole outer steps
    while ((kMinChunk << p->sub_shift) < chunk_bytes) ++p->sub_shift;

    // scratch kept per thread: a plan is built per batch, fresh pages every time would cost
    // more than filling them
    static thread_local std::vector<Piece> pieces;
    pieces.clear();
    for (const Span& sp : spans) {
      if (sp.group == 0) {
        for (uint64_t o = 0; o < sp.bytes; o += chunk_bytes)
          pieces.push_back(Piece{sp.src + o, sp.dst + o, sp.packed + o,
                                 static_cast<uint32_t>(std::min<uint64_t>(chunk_bytes, sp.bytes - o)),
                                 sp.tensor, 0, 0});
      } else {
        const uint64_t steps_per = chunk_bytes / sp.group;
        const uint64_t per = steps_per * sp.group;
        for (uint64_t o = 0, step = 0; o < sp.bytes; o += per, step += steps_per) {
          pieces.push_back(Piece{sp.src + step * sp.s_outer, sp.dst + step * sp.d_outer,
                                 sp.packed + o,
                                 static_cast<uint32_t>(std::min<uint64_t>(per, sp.bytes - o)),
                                 sp.tensor, 0, sp.shape});
          ++p->n_strided;
        }
      }
    }
    if (int rc = finish_plan(p.get(), pieces)) return rc;
    *out = p.release();
    return KVT_OK;
  });
}

uint64_t kvt_plan_num_strided_chunks(const kvt_plan* p) { return p ? p->n_strided : 0; }

int kvt_plan_host_tables(const kvt_plan* p, const void** chunks, uint64_t* n_chunks,
                         uint32_t* chunk_bytes, const void** shapes) {
  if (!p || !chunks || !n_chunks || !chunk_bytes || !shapes)
    return fail(KVT_ERR_INVALID, "kvt_plan_host_tables: null argument");
  if (p->device != KVT_DEVICE_NONE)
    return fail(KVT_ERR_INVALID, "kvt_plan_host_tables: the plan lives on a device");
  *chunks = p->host_table.data();
  *n_chunks = p->n_chunks;
  *chunk_bytes = kMinChunk << p->sub_shift;
  *shapes = &p->shapes;
  return KVT_OK;
}

void kvt_plan_destroy(kvt_plan* p) {
  if (!p) return;
  if (p->uploaded) {
    (void)hipEventSynchronize(p->uploaded);  // the upload reads the pinned twin
    (void)hipEventDestroy(p->uploaded);
  }
  table_pool().release(p->buf);
  delete p;
}

int kvt_plan_ready(const kvt_plan* p) {
  return guarded([&]() -> int {
    if (!p) return fail(KVT_ERR_INVALID, "kvt_plan_ready: null plan");
    if (p->uploaded && !p->upload_seen) {
      KVT_HIP(hipEventSynchronize(p->uploaded));
      p->upload_seen = true;
    }
    return KVT_OK;
  });
}

uint32_t kvt_plan_num_tensors(const kvt_plan* p) { return p ? p->n_tensors : 0; }
uint64_t kvt_plan_num_chunks(const kvt_plan* p) { return p ? p->n_chunks : 0; }
uint64_t kvt_plan_tensor_bytes(const kvt_plan* p, uint32_t t) {
  return (p && t < p->n_tensors) ? p->tensor_bytes[t] : 0;
}
uint64_t kvt_plan_tensor_offset(const kvt_plan* p, uint32_t t) {
  return (p && t < p->n_tensors) ? p->tensor_offset[t] : 0;
}
uint64_t kvt_plan_layer_bytes(const kvt_plan* p) { return p ? p->layer_bytes : 0; }

static int run_plan(bool pack, const kvt_plan* p, const kvt_cache* cache, uint32_t first_layer,
                    uint32_t n_layers, void* packed, uint64_t layer_stride, void* stream,
                    const uint64_t* blob_offsets = nullptr) {
  if (!p || !cache || (!packed && p->n_chunks))
    return fail(KVT_ERR_INVALID, "kvt_pack/unpack: null argument");
  if (p->device == KVT_DEVICE_NONE) return fail(KVT_ERR_INVALID, "a host-only plan cannot be launched");
  if (p->device != cache->device) return fail(KVT_ERR_INVALID, "plan and cache are on different devices");
  if (p->n_tensors != cache->n_tensors)
    return fail(KVT_ERR_INVALID, "plan and cache disagree on tensors per layer");
  if (static_cast<uint64_t>(first_layer) + n_layers > cache->n_layers)
    return fail(KVT_ERR_OUT_OF_RANGE, "layer range exceeds the registered cache");
  if (n_layers > 65535) return fail(KVT_ERR_INVALID, "at most 65535 layers per launch");
  if (n_layers > 1 && !blob_offsets && layer_stride < p->layer_bytes)
    return fail(KVT_ERR_INVALID, "layer_stride smaller than one packed layer");
  BlobOffsets blobs{};
  for (uint32_t t = 0; t < p->n_tensors; ++t)
    blobs.off[t] = blob_offsets ? blob_offsets[t] : p->tensor_offset[t];
  if (p->xform && (blobs.off[0] & 15u))
    return fail(KVT_ERR_INVALID, "layout transform needs a 16-byte aligned blob offset");
  const std::vector<uint64_t>& need = pack ? p->src_cap : p->dst_cap;
  for (uint32_t t = 0; t < p->n_tensors; ++t)
    if (cache->capacity[t] < need[t])
      return fail(KVT_ERR_OUT_OF_RANGE, "registered cache is smaller than the plan's capacity");
  DeviceGuard g;
  if (int rc = g.enter(p->device)) return rc;
  const hipStream_t s = static_cast<hipStream_t>(stream);
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &cap) != hipSuccess) (void)hipGetLastError();
  const bool capturing = cap != hipStreamCaptureStatusNone;
  if (p->uploaded && !p->upload_seen) {
    if (capturing)  // event queries and waits on outside events are not allowed inside a capture
      return fail(KVT_ERR_INVALID,
                  "the plan's table upload has not been observed yet: call kvt_plan_ready() "
                  "before using the plan inside a stream capture");
    if (hipEventQuery(p->uploaded) == hipSuccess) {
      p->upload_seen = true;
    } else {
      (void)hipGetLastError();
      KVT_HIP(hipStreamWaitEvent(s, p->uploaded, 0));
    }
  }
  const Chunk* table = p->dev_chunks + (pack ? 0 : p->n_chunks);
  const uint32_t n = static_cast<uint32_t>(p->n_chunks);
  if (p->strided) {
    if ((reinterpret_cast<uintptr_t>(packed) | layer_stride) & 15u)
      return fail(KVT_ERR_INVALID, "a strided plan needs a 16-byte aligned packed buffer and stride");
    for (uint32_t t = 0; t < p->n_tensors; ++t)
      if (blobs.off[t] & 15u)
        return fail(KVT_ERR_INVALID, "a strided plan needs 16-byte aligned blob offsets");
    if (!cache->aligned16)
      return fail(KVT_ERR_INVALID, "a strided plan needs 16-byte aligned layer tensors");
  }
  const hipError_t e =
      p->strided ? launch_strided_chunks(pack, table, n, p->sub_shift, cache->dev_ptrs,
                                         p->n_tensors, first_layer, n_layers,
                                         static_cast<uint8_t*>(packed), layer_stride, blobs,
                                         p->shapes, s) :
      p->xform ? launch_xform_chunks(pack, table, n, p->sub_shift, cache->dev_ptrs, p->n_tensors,
                                     first_layer, n_layers, static_cast<uint8_t*>(packed),
                                     layer_stride, blobs, p->xdev, s)
               : launch_copy_chunks(pack, table, n, p->sub_shift, cache->dev_ptrs, p->n_tensors,
                                    first_layer, n_layers, static_cast<uint8_t*>(packed),
                                    layer_stride, blobs, s);
  if (e != hipSuccess) return hip_fail(e, pack ? "pack launch" : "unpack launch");
  if (p->buf) {
    // remember when the table is last read, so that its storage is not recycled too early
    if (capturing) {
      p->buf->captured = true;
    } else {
      KVT_HIP(hipEventRecord(p->buf->last_use, s));
      p->buf->used = true;
    }
  }
  return KVT_OK;
}

int kvt_pack(const kvt_plan* p, const kvt_cache* cache, uint32_t first_layer, uint32_t n_layers,
             void* packed, uint64_t layer_stride, void* stream) {
  return guarded([&]() { return run_plan(true, p, cache, first_layer, n_layers, packed, layer_stride, stream); });
}

int kvt_unpack(const kvt_plan* p, const kvt_cache* cache, uint32_t first_layer, uint32_t n_layers,
               const void* packed, uint64_t layer_stride, void* stream) {
  return guarded([&]() {
    return run_plan(false, p, cache, first_layer, n_layers, const_cast<void*>(packed), layer_stride, stream);
  });
}

int kvt_pack_at(const kvt_plan* p, const kvt_cache* cache, uint32_t first_layer, uint32_t n_layers,
                void* base, uint64_t layer_stride, const uint64_t* blob_offsets, void* stream) {
  return guarded([&]() {
    return run_plan(true, p, cache, first_layer, n_layers, base, layer_stride, stream, blob_offsets);
  });
}

int kvt_unpack_at(const kvt_plan* p, const kvt_cache* cache, uint32_t first_layer,
                  uint32_t n_layers, const void* base, uint64_t layer_stride,
                  const uint64_t* blob_offsets, void* stream) {
  return guarded([&]() {
    return run_plan(false, p, cache, first_layer, n_layers, const_cast<void*>(base), layer_stride,
                    stream, blob_offsets);
  });
}

// ------------------------------------------- reference-shaped entry points

static int range_launch_shape(int64_t n, int num_wg, int* wgs) {
  if (n > 0x7FFFFFFFll) return fail(KVT_ERR_INVALID, "too many ranges");
  int w = num_wg > 0 ? num_wg : static_cast<int>(std::min<int64_t>(n, 1 << 20));
  *wgs = std::max(1, w);
  return KVT_OK;
}

static int launch_ranges(bool convert, const void* src, void* dst, const int64_t* so,
                         const int64_t* dof, const int64_t* len, int64_t n, int num_wg,
                         int threads_per_wg, void* stream) {
  (void)threads_per_wg;  // workgroups are always 256 lanes (4 wavefronts)
  if (n == 0) return KVT_OK;
  if (n < 0 || !src || !dst || !so || !dof || !len)
    return fail(KVT_ERR_INVALID, "launch_copy: bad argument");
  if (usable_devices() <= 0) return fail(KVT_ERR_NO_DEVICE, "no usable gfx950 (MI355X) device");
  int wgs = 0;
  if (int rc = range_launch_shape(n, num_wg, &wgs)) return rc;
  // The range lengths live on the device; eight workgroups stride over each range's slices.
  const int rows = 8;
  const hipStream_t s = static_cast<hipStream_t>(stream);
  const hipError_t e = convert ? launch_convert_ranges(src, dst, so, dof, len, n, wgs, rows, s)
                               : launch_copy_ranges(src, dst, so, dof, len, n, wgs, rows, s);
  if (e != hipSuccess) return hip_fail(e, "range copy launch");
  return KVT_OK;
}

int kvt_launch_copy_d2h_direct(const void* gpu_src_base, void* dst, const int64_t* src_offsets,
                               const int64_t* dst_offsets, const int64_t* lengths, int64_t n,
                               int num_wg, int threads_per_wg, void* stream) {
  return guarded([&]() {
    return launch_ranges(false, gpu_src_base, dst, src_offsets, dst_offsets, lengths, n, num_wg,
                         threads_per_wg, stream);
  });
}

int kvt_launch_copy_h2d_direct(const void* src, void* gpu_dst_base, const int64_t* src_offsets,
                               const int64_t* dst_offsets, const int64_t* lengths, int64_t n,
                               int num_wg, int threads_per_wg, void* stream) {
  return guarded([&]() {
    return launch_ranges(false, src, gpu_dst_base, src_offsets, dst_offsets, lengths, n, num_wg,
                         threads_per_wg, stream);
  });
}

int kvt_launch_copy_d2h_bf16_to_fp8(const void* gpu_src_base, void* dst,
                                    const int64_t* src_offsets, const int64_t* dst_offsets,
                                    const int64_t* lengths, int64_t n, int num_wg,
                                    int threads_per_wg, void* stream) {
  return guarded([&]() {
    return launch_ranges(true, gpu_src_base, dst, src_offsets, dst_offsets, lengths, n, num_wg,
                         threads_per_wg, stream);
  });
}

// Shared body of the two "handle data" entry points. `halve`: converting
// gather (contiguous side advances by length / 2, lengths passed to the kernel
// are element counts).
static int handle_data(void* tensor_buf, void* layer_gpu_ptr, const kvt_ipc_block* blocks,
                       uint64_t n, uint64_t tensor_data_size, int direction, bool halve,
                       int device, void* stream, int64_t* dev_meta, int64_t* host_meta,
                       int64_t max_block_num) {
  if (n == 0) return KVT_OK;
  if (!tensor_buf || !layer_gpu_ptr || !blocks || !dev_meta || !host_meta)
    return fail(KVT_ERR_INVALID, "copy_handle_data: null argument");
  if (direction != KVT_COPY_H2D && direction != KVT_COPY_D2H)
    return fail(KVT_ERR_INVALID, "copy_handle_data: bad direction");
  if (int rc = check_device(device)) return rc;
  if (max_block_num <= 0) max_block_num = 8192;
  uint64_t total = 0;
  for (uint64_t i = 0; i < n; ++i) {
    if (blocks[i].length == 0) return fail(KVT_ERR_INVALID, "copy_handle_data: zero-length range");
    if (halve && (blocks[i].length & 1)) return fail(KVT_ERR_INVALID, "odd bf16 byte length");
    total += blocks[i].length;
  }
  if (total != tensor_data_size)
    return fail(KVT_ERR_INVALID, "copy_handle_data: tensor_data_size != sum of range lengths");
  DeviceGuard g;
  if (int rc = g.enter(device)) return rc;
  const hipStream_t s = static_cast<hipStream_t>(stream);
  uint64_t host_cursor = 0;
  for (uint64_t first = 0; first < n; first += static_cast<uint64_t>(max_block_num)) {
    const uint64_t m = std::min<uint64_t>(static_cast<uint64_t>(max_block_num), n - first);
    int64_t* contig = host_meta;
    int64_t* gpu = host_meta + m;
    int64_t* lens = host_meta + 2 * m;
    uint64_t longest = 0;
    for (uint64_t i = 0; i < m; ++i) {
      const kvt_ipc_block& b = blocks[first + i];
      contig[i] = static_cast<int64_t>(host_cursor);
      gpu[i] = static_cast<int64_t>(b.dst_offset);
      lens[i] = static_cast<int64_t>(halve ? b.length / 2 : b.length);
      host_cursor += halve ? b.length / 2 : b.length;
      longest = std::max<uint64_t>(longest, b.length);
    }
    KVT_HIP(hipMemcpyAsync(dev_meta, host_meta, 3 * m * sizeof(int64_t), hipMemcpyHostToDevice, s));
    const int64_t* d_contig = dev_meta;
    const int64_t* d_gpu = dev_meta + m;
    const int64_t* d_lens = dev_meta + 2 * m;
    const int wgs = static_cast<int>(m);
    // one workgroup per 4 KiB slice of the longest range (bounded; longer ranges are strided)
    const uint64_t unit = halve ? 8192 : 4096;
    const int rows = static_cast<int>(std::min<uint64_t>(std::max<uint64_t>(1, (longest + unit - 1) / unit), 512));
    hipError_t e;
    if (halve)
      e = launch_convert_ranges(layer_gpu_ptr, tensor_buf, d_gpu, d_contig, d_lens,
                                static_cast<int64_t>(m), wgs, rows, s);
    else if (direction == KVT_COPY_D2H)
      e = launch_copy_ranges(layer_gpu_ptr, tensor_buf, d_gpu, d_contig, d_lens,
                             static_cast<int64_t>(m), wgs, rows, s);
    else
      e = launch_copy_ranges(tensor_buf, layer_gpu_ptr, d_contig, d_gpu, d_lens,
                             static_cast<int64_t>(m), wgs, rows, s);
    if (e != hipSuccess) return hip_fail(e, "copy_handle_data launch");
    // the metadata buffers are reused by the next batch
    if (first + m < n) KVT_HIP(hipStreamSynchronize(s));
  }
  return KVT_OK;
}

int kvt_copy_handle_data_with_kernel(void* tensor_buf, void* layer_gpu_ptr,
                                     const kvt_ipc_block* blocks, uint64_t n,
                                     uint64_t tensor_data_size, int direction, int device,
                                     void* stream, int64_t* dev_meta, int64_t* host_meta,
                                     int64_t max_block_num) {
  return guarded([&]() {
    return handle_data(tensor_buf, layer_gpu_ptr, blocks, n, tensor_data_size, direction, false,
                       device, stream, dev_meta, host_meta, max_block_num);
  });
}

int kvt_copy_d2h_bf16_to_fp8(void* tensor_buf, const void* layer_gpu_ptr,
                             const kvt_ipc_block* blocks, uint64_t n, uint64_t tensor_data_size,
                             int device, void* stream, int64_t* dev_meta, int64_t* host_meta,
                             int64_t max_block_num) {
  return guarded([&]() {
    return handle_data(tensor_buf, const_cast<void*>(layer_gpu_ptr), blocks, n, tensor_data_size,
                       KVT_COPY_D2H, true, device, stream, dev_meta, host_meta, max_block_num);
  });
}

// ----------------------------------------------------------------- session

int kvt_session_create(const kvt_plan* plan, const kvt_cache* cache, void* packed,
                       uint64_t layer_stride, kvt_session** out) {
  return guarded([&]() -> int {
    if (!plan || !cache || !packed || !out)
      return fail(KVT_ERR_INVALID, "kvt_session_create: null argument");
    if (layer_stride < plan->layer_bytes)
      return fail(KVT_ERR_INVALID, "kvt_session_create: layer_stride smaller than one packed layer");
    if (int rc = check_device(plan->device)) return rc;
    DeviceGuard g;
    if (int rc = g.enter(plan->device)) return rc;
    if (int rc = kvt_plan_ready(plan)) return rc;  // save_layer may run inside a stream capture
    std::unique_ptr<kvt_session> s(new kvt_session());
    s->plan = plan;
    s->cache = cache;
    s->packed = packed;
    s->layer_stride = layer_stride;
    KVT_HIP(hipStreamCreateWithFlags(&s->side, hipStreamNonBlocking));
    s->ready.resize(cache->n_layers);
    s->done.resize(cache->n_layers);
    s->issued.assign(cache->n_layers, 0);
    for (uint32_t l = 0; l < cache->n_layers; ++l) {
      KVT_HIP(hipEventCreateWithFlags(&s->ready[l], hipEventDisableTiming));
      KVT_HIP(hipEventCreateWithFlags(&s->done[l], hipEventDisableTiming));
    }
    *out = s.release();
    return KVT_OK;
  });
}

void kvt_session_destroy(kvt_session* s) {
  if (!s) return;
  if (s->side) {
    (void)hipStreamSynchronize(s->side);
    (void)hipStreamDestroy(s->side);
  }
  for (hipEvent_t e : s->ready)
    if (e) (void)hipEventDestroy(e);
  for (hipEvent_t e : s->done)
    if (e) (void)hipEventDestroy(e);
  delete s;
}

int kvt_session_save_layer(kvt_session* s, uint32_t layer, void* compute_stream) {
  return guarded([&]() -> int {
    if (!s) return fail(KVT_ERR_INVALID, "kvt_session_save_layer: null session");
    if (layer >= s->cache->n_layers) return fail(KVT_ERR_OUT_OF_RANGE, "layer out of range");
    DeviceGuard g;
    if (int rc = g.enter(s->plan->device)) return rc;
    KVT_HIP(hipEventRecord(s->ready[layer], static_cast<hipStream_t>(compute_stream)));
    KVT_HIP(hipStreamWaitEvent(s->side, s->ready[layer], 0));
    uint8_t* dst = static_cast<uint8_t*>(s->packed) + static_cast<uint64_t>(layer) * s->layer_stride;
    if (int rc = run_plan(true, s->plan, s->cache, layer, 1, dst, s->layer_stride, s->side)) return rc;
    KVT_HIP(hipEventRecord(s->done[layer], s->side));
    {
      std::lock_guard<std::mutex> lock(s->mu);
      s->last_done = s->done[layer];
      s->issued[layer] = 1;
    }
    s->issued_cv.notify_all();
    return KVT_OK;
  });
}

int kvt_session_wait_layer(kvt_session* s, uint32_t layer) {
  return guarded([&]() -> int {
    if (!s) return fail(KVT_ERR_INVALID, "kvt_session_wait_layer: null session");
    if (layer >= s->cache->n_layers) return fail(KVT_ERR_OUT_OF_RANGE, "layer out of range");
    {
      std::unique_lock<std::mutex> lock(s->mu);
      s->issued_cv.wait(lock, [&] { return s->issued[layer] != 0; });
    }
    KVT_HIP(hipEventSynchronize(s->done[layer]));
    return KVT_OK;
  });
}

int kvt_session_join(kvt_session* s, void* stream) {
  return guarded([&]() -> int {
    if (!s) return fail(KVT_ERR_INVALID, "kvt_session_join: null session");
    if (s->last_done) KVT_HIP(hipStreamWaitEvent(static_cast<hipStream_t>(stream), s->last_done, 0));
    return KVT_OK;
  });
}

void* kvt_session_side_stream(kvt_session* s) { return s ? s->side : nullptr; }

// ------------------------------------------------------------------ stager

int kvt_stager_create(int device, uint64_t slot_bytes, uint32_t n_slots, kvt_stager** out) {
  return guarded([&]() -> int {
    if (!out || slot_bytes == 0 || n_slots < 2)
      return fail(KVT_ERR_INVALID, "kvt_stager_create: need >= 2 slots of > 0 bytes");
    if (int rc = check_device(device)) return rc;
    DeviceGuard g;
    if (int rc = g.enter(device)) return rc;
    std::unique_ptr<kvt_stager> s(new kvt_stager());
    s->device = device;
    s->slot_bytes = round_up(slot_bytes, 4096);
    s->n_slots = n_slots;
    KVT_HIP(hipHostMalloc(reinterpret_cast<void**>(&s->pinned), s->slot_bytes * n_slots,
                          hipHostMallocDefault));
    KVT_HIP(hipStreamCreateWithFlags(&s->copy, hipStreamNonBlocking));
    s->slot_done.resize(n_slots);
    for (uint32_t i = 0; i < n_slots; ++i)
      KVT_HIP(hipEventCreateWithFlags(&s->slot_done[i], hipEventDisableTiming));
    KVT_HIP(hipEventCreateWithFlags(&s->fence, hipEventDisableTiming));
    *out = s.release();
    return KVT_OK;
  });
}

void kvt_stager_destroy(kvt_stager* s) {
  if (!s) return;
  if (s->copy) {
    (void)hipStreamSynchronize(s->copy);
    (void)hipStreamDestroy(s->copy);
  }
  for (hipEvent_t e : s->slot_done)
    if (e) (void)hipEventDestroy(e);
  if (s->fence) (void)hipEventDestroy(s->fence);
  if (s->pinned) (void)hipHostFree(s->pinned);
  delete s;
}

void* kvt_stager_slot(kvt_stager* s, uint32_t slot) {
  return (s && slot < s->n_slots) ? s->pinned + static_cast<uint64_t>(slot) * s->slot_bytes : nullptr;
}
void* kvt_stager_copy_stream(kvt_stager* s) { return s ? s->copy : nullptr; }

int kvt_stager_save(kvt_stager* s, uint32_t slot, const void* dev, uint64_t bytes,
                    void* producer_stream) {
  return kvt_stager_save_at(s, slot, 0, dev, bytes, producer_stream);
}

int kvt_stager_save_at(kvt_stager* s, uint32_t slot, uint64_t slot_offset, const void* dev,
                       uint64_t bytes, void* producer_stream) {
  return guarded([&]() -> int {
    if (!s || !dev) return fail(KVT_ERR_INVALID, "kvt_stager_save: null argument");
    if (slot >= s->n_slots || slot_offset > s->slot_bytes || bytes > s->slot_bytes - slot_offset)
      return fail(KVT_ERR_OUT_OF_RANGE, "kvt_stager_save: slot index or size out of range");
    DeviceGuard g;
    if (int rc = g.enter(s->device)) return rc;
    KVT_HIP(hipEventRecord(s->fence, static_cast<hipStream_t>(producer_stream)));
    KVT_HIP(hipStreamWaitEvent(s->copy, s->fence, 0));
    KVT_HIP(hipMemcpyAsync(static_cast<uint8_t*>(kvt_stager_slot(s, slot)) + slot_offset, dev, bytes,
                           hipMemcpyDeviceToHost, s->copy));
    KVT_HIP(hipEventRecord(s->slot_done[slot], s->copy));
    return KVT_OK;
  });
}

int kvt_stager_load(kvt_stager* s, uint32_t slot, void* dev, uint64_t bytes,
                    void* consumer_stream) {
  return kvt_stager_load_at(s, slot, 0, dev, bytes, consumer_stream);
}

int kvt_stager_load_at(kvt_stager* s, uint32_t slot, uint64_t slot_offset, void* dev,
                       uint64_t bytes, void* consumer_stream) {
  return guarded([&]() -> int {
    if (!s || !dev) return fail(KVT_ERR_INVALID, "kvt_stager_load: null argument");
    if (slot >= s->n_slots || slot_offset > s->slot_bytes || bytes > s->slot_bytes - slot_offset)
      return fail(KVT_ERR_OUT_OF_RANGE, "kvt_stager_load: slot index or size out of range");
    DeviceGuard g;
    if (int rc = g.enter(s->device)) return rc;
    // the device buffer may still be read by earlier work of the consumer
    KVT_HIP(hipEventRecord(s->fence, static_cast<hipStream_t>(consumer_stream)));
    KVT_HIP(hipStreamWaitEvent(s->copy, s->fence, 0));
    KVT_HIP(hipMemcpyAsync(dev, static_cast<uint8_t*>(kvt_stager_slot(s, slot)) + slot_offset, bytes,
                           hipMemcpyHostToDevice, s->copy));
    KVT_HIP(hipEventRecord(s->slot_done[slot], s->copy));
    KVT_HIP(hipStreamWaitEvent(static_cast<hipStream_t>(consumer_stream), s->slot_done[slot], 0));
    return KVT_OK;
  });
}

int kvt_stager_wait(kvt_stager* s, uint32_t slot) {
  return guarded([&]() -> int {
    if (!s || slot >= s->n_slots) return fail(KVT_ERR_INVALID, "kvt_stager_wait: bad argument");
    KVT_HIP(hipEventSynchronize(s->slot_done[slot]));
    return KVT_OK;
  });
}

int kvt_measure_pcie(int device, int direction, uint64_t bytes, uint32_t repeats,
                     double* bytes_per_s) {
  return guarded([&]() -> int {
    if (!bytes_per_s || bytes == 0 || repeats == 0)
      return fail(KVT_ERR_INVALID, "kvt_measure_pcie: bad argument");
    if (int rc = check_device(device)) return rc;
    DeviceGuard g;
    if (int rc = g.enter(device)) return rc;
    void *host = nullptr, *dev = nullptr;
    hipStream_t st = nullptr;
    hipEvent_t a = nullptr, b = nullptr;
    int rc = KVT_OK;
    auto cleanup = [&]() {
      if (a) (void)hipEventDestroy(a);
      if (b) (void)hipEventDestroy(b);
      if (st) (void)hipStreamDestroy(st);
      if (dev) (void)hipFree(dev);
      if (host) (void)hipHostFree(host);
    };
#define KVT_TRY(call)                         \
  do {                                        \
    const hipError_t _e = (call);             \
    if (_e != hipSuccess) {                   \
      rc = hip_fail(_e, #call);               \
      cleanup();                              \
      return rc;                              \
    }                                         \
  } while (0)
    KVT_TRY(hipHostMalloc(&host, bytes, hipHostMallocDefault));
    KVT_TRY(hipMalloc(&dev, bytes));
    std::memset(host, 0x5a, bytes);
    KVT_TRY(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
    KVT_TRY(hipEventCreate(&a));
    KVT_TRY(hipEventCreate(&b));
    const bool d2h = direction == KVT_COPY_D2H;
    KVT_TRY(hipMemcpyAsync(d2h ? host : dev, d2h ? dev : host, bytes,
                           d2h ? hipMemcpyDeviceToHost : hipMemcpyHostToDevice, st));
    KVT_TRY(hipEventRecord(a, st));
    for (uint32_t i = 0; i < repeats; ++i)
      KVT_TRY(hipMemcpyAsync(d2h ? host : dev, d2h ? dev : host, bytes,
                             d2h ? hipMemcpyDeviceToHost : hipMemcpyHostToDevice, st));
    KVT_TRY(hipEventRecord(b, st));
    KVT_TRY(hipEventSynchronize(b));
    float ms = 0;
    KVT_TRY(hipEventElapsedTime(&ms, a, b));
#undef KVT_TRY
    *bytes_per_s = static_cast<double>(bytes) * repeats / (ms * 1e-3);
    cleanup();
    return KVT_OK;
  });
}

// --------------------------------------------------------------- utilities

int kvt_copy_linear(void* dst, const void* src, uint64_t bytes, void* stream) {
  return guarded([&]() -> int {
    if ((!dst || !src) && bytes) return fail(KVT_ERR_INVALID, "kvt_copy_linear: null argument");
    if (usable_devices() <= 0) return fail(KVT_ERR_NO_DEVICE, "no usable gfx950 (MI355X) device");
    if (bytes > (0x7FFFFFF0ull << 12)) return fail(KVT_ERR_INVALID, "kvt_copy_linear: too large");
    const hipError_t e = launch_copy_linear(dst, src, bytes, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "linear copy launch");
    return KVT_OK;
  });
}

int kvt_event_create(void** ev) {
  if (!ev) return fail(KVT_ERR_INVALID, "kvt_event_create: null argument");
  if (usable_devices() <= 0) return fail(KVT_ERR_NO_DEVICE, "no usable gfx950 (MI355X) device");
  hipEvent_t e;
  KVT_HIP(hipEventCreate(&e));
  *ev = e;
  return KVT_OK;
}
int kvt_event_destroy(void* ev) {
  if (ev) KVT_HIP(hipEventDestroy(static_cast<hipEvent_t>(ev)));
  return KVT_OK;
}
int kvt_event_record(void* ev, void* stream) {
  KVT_HIP(hipEventRecord(static_cast<hipEvent_t>(ev), static_cast<hipStream_t>(stream)));
  return KVT_OK;
}
int kvt_event_synchronize(void* ev) {
  KVT_HIP(hipEventSynchronize(static_cast<hipEvent_t>(ev)));
  return KVT_OK;
}
int kvt_event_elapsed_ms(void* start, void* stop, float* ms) {
  if (!ms) return fail(KVT_ERR_INVALID, "kvt_event_elapsed_ms: null argument");
  KVT_HIP(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
  return KVT_OK;
}
int kvt_stream_create(void** stream) {
  if (!stream) return fail(KVT_ERR_INVALID, "kvt_stream_create: null argument");
  if (usable_devices() <= 0) return fail(KVT_ERR_NO_DEVICE, "no usable gfx950 (MI355X) device");
  hipStream_t s;
  KVT_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  *stream = s;
  return KVT_OK;
}
int kvt_stream_destroy(void* stream) {
  if (stream) KVT_HIP(hipStreamDestroy(static_cast<hipStream_t>(stream)));
  return KVT_OK;
}
int kvt_stream_synchronize(void* stream) {
  KVT_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  return KVT_OK;
}

}  // extern "C"
