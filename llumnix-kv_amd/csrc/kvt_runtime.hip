// Device selection, the chunk-table pool, cache registration and the small
// event / stream utilities of the C ABI.
#include <algorithm>
#include <atomic>
#include <cstring>
#include <memory>

#include "kvt_runtime.h"

namespace kvt {

int hip_fail(hipError_t e, const char* what) {
  return fail(KVT_ERR_HIP, std::string(what) + ": " + hipGetErrorString(e));
}

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

// Share of the device a copy launch may occupy. A 256-lane workgroup is four wavefronts and
// a CU holds 32, so usage x CUs x 8 workgroups are resident at once on that share; a launch
// capped to that many (persistent, striding over the work) leaves the rest of the CUs to
// whatever else runs. Stored as the cap itself; 0 = one workgroup per slice, no limit.
constexpr int kMaxDevices = 64;
constexpr uint32_t kWgsPerCu = 8;
static std::atomic<uint32_t> g_wg_cap[kMaxDevices];
static std::atomic<uint64_t> g_usage_bits[kMaxDevices];   // the double as given; 0 = never set

uint32_t copy_wg_cap(int device) {
  return device >= 0 && device < kMaxDevices ? g_wg_cap[device].load(std::memory_order_relaxed) : 0;
}

uint32_t device_cu_count(int device) {
  static std::atomic<uint32_t> cached[kMaxDevices];
  if (device < 0 || device >= kMaxDevices) return 0;
  uint32_t n = cached[device].load(std::memory_order_relaxed);
  if (n == 0) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) {
      (void)hipGetLastError();
      return 0;
    }
    n = cus > 0 ? static_cast<uint32_t>(cus) : 0u;
    cached[device].store(n, std::memory_order_relaxed);
  }
  return n;
}

static std::atomic<uint64_t> g_cached_load_max{kTemporalMaxBytes};
uint64_t copy_cached_load_max_bytes() { return g_cached_load_max.load(std::memory_order_relaxed); }
static std::atomic<uint64_t> g_cached_store_max{0};
uint64_t copy_cached_store_max_bytes() { return g_cached_store_max.load(std::memory_order_relaxed); }

// A kernel that runs past a buffer takes a GPU memory fault, which can cost the whole
// process (and more) instead of an error code. What the runtime knows about a pointer is
// therefore checked on the host before a launch uses it: it must be memory the device can
// address, and where the runtime can name the allocation around it, [ptr, ptr + bytes) must
// lie inside. A framework's caching allocator hands out pieces of larger allocations, so this
// catches an extent that overshoots the underlying allocation, not one that overshoots the
// tensor. Spans that passed are remembered per thread (a serving loop reuses its buffers),
// so the steady state costs a few comparisons and no runtime call; an entry is trusted for
// 256 uses and then asked for again, since the memory behind an address can change hands.
static std::atomic<uint64_t> g_span_epoch{1};
void forget_device_spans() { g_span_epoch.fetch_add(1, std::memory_order_relaxed); }

int check_device_span(const void* ptr, uint64_t bytes, const std::string& what, bool* host_memory) {
  if (host_memory) *host_memory = false;
  if (bytes == 0) return KVT_OK;
  struct Span {
    uintptr_t lo = 0, hi = 0;
    unsigned uses = 0;
    uint64_t epoch = 0;
    bool host = false;
  };
  // Allocations the runtime has answered for lately, per thread: a lookup costs microseconds
  // and the same few buffers come back launch after launch. An answer is trusted for a bounded
  // number of uses and dropped as soon as the library itself frees device memory.
  static thread_local Span seen[8];
  static thread_local unsigned next = 0;
  const uintptr_t p = reinterpret_cast<uintptr_t>(ptr);
  const uint64_t epoch = g_span_epoch.load(std::memory_order_relaxed);
  for (Span& s : seen)
    if (s.epoch == epoch && p >= s.lo && p < s.hi && bytes <= s.hi - p) {
      if (host_memory) *host_memory = s.host;
      if (++s.uses < 256) return KVT_OK;
      s = Span{};  // ask the runtime again below
      break;
    }
  hipPointerAttribute_t attr{};
  if (hipPointerGetAttributes(&attr, ptr) != hipSuccess) {
    (void)hipGetLastError();
    return fail(KVT_ERR_INVALID, what + " is not memory the device can address");
  }
  if (attr.type == hipMemoryTypeUnregistered)
    return fail(KVT_ERR_INVALID, what + " is plain host memory the device cannot address");
  if (host_memory) *host_memory = attr.type == hipMemoryTypeHost;
  hipDeviceptr_t base = nullptr;
  size_t size = 0;
  if (hipMemGetAddressRange(&base, &size, const_cast<void*>(ptr)) != hipSuccess) {
    (void)hipGetLastError();  // pinned host memory, virtual-memory mappings: nothing to compare
    return KVT_OK;
  }
  const uintptr_t lo = reinterpret_cast<uintptr_t>(base);
  if (p < lo || p - lo > size || bytes > size - (p - lo))
    return fail(KVT_ERR_OUT_OF_RANGE,
                what + ": " + std::to_string(bytes) +
                    " bytes reach beyond the allocation that holds the pointer (" +
                    std::to_string(p < lo || p - lo > size ? 0 : size - (p - lo)) + " bytes left)");
  seen[next++ % 8] = Span{lo, lo + size, 0, epoch, attr.type == hipMemoryTypeHost};
  return KVT_OK;
}

TicketPool& ticket_pool() {
  static TicketPool* pool = new TicketPool();  // intentionally leaked, like the table pool
  return *pool;
}

TicketPool::PerDevice* TicketPool::of(int device) {
  if (device < 0) return nullptr;
  if (device >= static_cast<int>(devices_.size())) devices_.resize(device + 1);
  return &devices_[device];
}

int TicketPool::prepare(int device) {
  std::lock_guard<std::mutex> lock(mu_);
  PerDevice* d = of(device);
  if (!d) return fail(KVT_ERR_INVALID, "ticket pool: bad device");
  if (d->arena) return KVT_OK;
  DeviceGuard g;
  if (int rc = g.enter(device)) return rc;
  uint8_t* arena = nullptr;
  KVT_HIP(hipMalloc(reinterpret_cast<void**>(&arena), static_cast<size_t>(kBlockBytes) * kBlocks));
  const hipError_t e = hipMemset(arena, 0, static_cast<size_t>(kBlockBytes) * kBlocks);
  if (e != hipSuccess) {
    (void)hipFree(arena);
    return hip_fail(e, "ticket pool: hipMemset");
  }
  d->done.assign(kBlocks, nullptr);
  d->state.assign(kBlocks, kFree);
  d->arena = arena;
  return KVT_OK;
}

uint32_t* TicketPool::acquire(int device, bool permanent) {
  std::lock_guard<std::mutex> lock(mu_);
  PerDevice* d = of(device);
  if (!d || !d->arena) return nullptr;
  if (permanent) {
    // For a launch that is being recorded into a stream capture: no runtime call may be made
    // here (an event query inside a capture can be refused, or end the capture), so these
    // launches have blocks of their own that are never lent to eager launches and are simply
    // free or taken.
    for (uint32_t probe = 0; probe < kBlocks - kEagerBlocks; ++probe) {
      const uint32_t i = kEagerBlocks + (d->capture_cursor + probe) % (kBlocks - kEagerBlocks);
      if (d->state[i] != kFree) continue;
      d->state[i] = kPermanent;
      d->capture_cursor = (i + 1 - kEagerBlocks) % (kBlocks - kEagerBlocks);
      ++d->counters[2];
      return reinterpret_cast<uint32_t*>(d->arena + static_cast<size_t>(i) * kBlockBytes);
    }
    ++d->counters[3];
    return nullptr;
  }
  // a few probes from where the last search ended: blocks come free in the order they were lent
  for (uint32_t probe = 0; probe < 32; ++probe) {
    const uint32_t i = (d->cursor + probe) % kEagerBlocks;
    if (d->state[i] == kPermanent || d->state[i] == kLent) continue;
    if (d->state[i] == kInFlight) {
      if (hipEventQuery(d->done[i]) != hipSuccess) {
        (void)hipGetLastError();
        continue;
      }
      d->state[i] = kFree;
    }
    if (!d->done[i] &&
        hipEventCreateWithFlags(&d->done[i], hipEventDisableTiming) != hipSuccess) {
      (void)hipGetLastError();
      d->done[i] = nullptr;
      ++d->counters[1];
      return nullptr;
    }
    d->state[i] = kLent;
    d->cursor = (i + 1) % kEagerBlocks;
    ++d->counters[0];
    return reinterpret_cast<uint32_t*>(d->arena + static_cast<size_t>(i) * kBlockBytes);
  }
  d->cursor = (d->cursor + 32) % kEagerBlocks;
  ++d->counters[1];
  return nullptr;
}

void TicketPool::stats(int device, uint64_t out[4]) {
  std::lock_guard<std::mutex> lock(mu_);
  PerDevice* d = of(device);
  for (int i = 0; i < 4; ++i) out[i] = d ? d->counters[i] : 0;
}

void TicketPool::launched(int device, uint32_t* block, hipStream_t stream) {
  std::lock_guard<std::mutex> lock(mu_);
  PerDevice* d = of(device);
  if (!d || !d->arena || !block) return;
  const size_t i = (reinterpret_cast<uint8_t*>(block) - d->arena) / kBlockBytes;
  // no event, no way to tell when the launch has ended: the block stays out of circulation
  if (i >= kBlocks) return;
  if (!d->done[i] || hipEventRecord(d->done[i], stream) != hipSuccess) {
    (void)hipGetLastError();
    d->state[i] = kPermanent;
    return;
  }
  d->state[i] = kInFlight;
}

void TicketPool::give_back(int device, uint32_t* block) {
  std::lock_guard<std::mutex> lock(mu_);
  PerDevice* d = of(device);
  if (!d || !d->arena || !block) return;
  const size_t i = (reinterpret_cast<uint8_t*>(block) - d->arena) / kBlockBytes;
  if (i < kBlocks && (d->state[i] == kPermanent || d->state[i] == kLent)) d->state[i] = kFree;
}

TablePool& table_pool() {
  static TablePool* pool = new TablePool();  // intentionally leaked: outlives static destruction
  return *pool;
}

}  // namespace kvt

using namespace kvt;

extern "C" {

int kvt_device_count(void) { return std::max(0, usable_devices()); }

int kvt_set_copy_cached_load_max(uint64_t payload_bytes) {
  g_cached_load_max.store(payload_bytes, std::memory_order_relaxed);
  return KVT_OK;
}
uint64_t kvt_get_copy_cached_load_max(void) { return copy_cached_load_max_bytes(); }
int kvt_set_copy_cached_store_max(uint64_t payload_bytes) {
  g_cached_store_max.store(payload_bytes, std::memory_order_relaxed);
  return KVT_OK;
}
uint64_t kvt_get_copy_cached_store_max(void) { return copy_cached_store_max_bytes(); }

int kvt_set_copy_cu_usage(int device, double usage) {
  return guarded([&]() -> int {
    if (int rc = check_device(device)) return rc;
    if (device >= kMaxDevices) return fail(KVT_ERR_INVALID, "kvt_set_copy_cu_usage: device index too large");
    if (!(usage > 0.0 && usage <= 1.0))
      return fail(KVT_ERR_INVALID, "kvt_set_copy_cu_usage: usage must be in (0, 1]");
    uint32_t cap = 0;
    if (usage < 1.0) {
      int cus = 0;
      KVT_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
      const double wgs = usage * static_cast<double>(cus) * kWgsPerCu;
      cap = std::max<uint32_t>(8u, static_cast<uint32_t>(wgs) & ~7u);
    }
    // the ticket blocks of the persistent kernels: allocated here, not inside a launch
    if (cap != 0)
      if (int rc = ticket_pool().prepare(device)) return rc;
    uint64_t bits = 0;
    std::memcpy(&bits, &usage, sizeof(bits));
    g_usage_bits[device].store(bits, std::memory_order_relaxed);
    g_wg_cap[device].store(cap, std::memory_order_relaxed);
    return KVT_OK;
  });
}

int kvt_get_copy_cu_usage(int device, double* usage, uint32_t* max_workgroups) {
  if (int rc = check_device(device)) return rc;
  if (device >= kMaxDevices) return fail(KVT_ERR_INVALID, "kvt_get_copy_cu_usage: device index too large");
  const uint64_t bits = g_usage_bits[device].load(std::memory_order_relaxed);
  if (usage) {
    *usage = 1.0;
    if (bits != 0) std::memcpy(usage, &bits, sizeof(bits));
  }
  if (max_workgroups) *max_workgroups = g_wg_cap[device].load(std::memory_order_relaxed);
  return KVT_OK;
}

int kvt_get_copy_ticket_stats(int device, uint64_t out[4]) {
  if (!out) return fail(KVT_ERR_INVALID, "kvt_get_copy_ticket_stats: null argument");
  if (int rc = check_device(device)) return rc;
  ticket_pool().stats(device, out);
  return KVT_OK;
}

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
      if (reinterpret_cast<uintptr_t>(ptrs[i]) & 3u) c->aligned4 = false;
      if (int rc = check_device_span(ptrs[i], capacity[i % n_tensors],
                                     "kvt_cache_register: layer " + std::to_string(i / n_tensors) +
                                         " tensor " + std::to_string(i % n_tensors)))
        return rc;
    }
    // at least one 16-byte vector long: idle lanes of a capped launch load from its start
    KVT_HIP(hipMalloc(reinterpret_cast<void**>(&c->dev_ptrs), std::max<uint64_t>(16, n * sizeof(void*))));
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
  forget_device_spans();  // the caller is about to free the tensors this cache named
  if (c->dev_ptrs) (void)hipFree(c->dev_ptrs);
  delete c;
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

int kvt_copy_runtime_d2d(void* dst, const void* src, uint64_t bytes, void* stream) {
  return guarded([&]() -> int {
    if ((!dst || !src) && bytes) return fail(KVT_ERR_INVALID, "kvt_copy_runtime_d2d: null argument");
    if (usable_devices() <= 0) return fail(KVT_ERR_NO_DEVICE, "no usable gfx950 (MI355X) device");
    if (bytes == 0) return KVT_OK;
    KVT_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, static_cast<hipStream_t>(stream)));
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
