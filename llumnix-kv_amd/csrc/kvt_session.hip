// Per-layer gating sessions (event -> side stream -> pack -> done event) and
// pinned-host staging of packed layers.
#include <algorithm>
#include <chrono>
#include <condition_variable>
#include <cstring>
#include <memory>
#include <string>
#include <thread>

#include "kvt_runtime.h"

using namespace kvt;

// Completion of a layer's pack is published by the device itself: a one-lane kernel behind
// the pack on the side stream bumps the layer's counter in device memory and mirrors it into
// pinned host memory. A host thread that waits for "the k-th pack of layer l" polls that
// word -- no event, no stream, no device-wide synchronisation -- so the signal is the same
// whether the sequence was issued eagerly or is replayed from a hipGraph, where a host-side
// event wait has nothing to hold on to.
struct kvt_session {
  const kvt_plan* plan = nullptr;
  const kvt_cache* cache = nullptr;
  void* packed = nullptr;
  uint64_t layer_stride = 0;
  hipStream_t side = nullptr;
  std::vector<hipEvent_t> ready;
  hipEvent_t joined = nullptr;     // recorded on the side stream by kvt_session_join
  hipEvent_t inline_done = nullptr;  // behind the last eager inline pack (on the caller's stream)
  bool inline_any = false;
  bool issued_any = false;
  uint32_t* count_dev = nullptr;   // per layer: packs completed so far (device memory)
  uint32_t* count_host = nullptr;  // the same, mirrored by the device into pinned host memory

  // Host bookkeeping of steps (one forward pass each). target[l] of a step = which completion
  // of layer l belongs to it (0 = not submitted yet); the last kSteps steps are kept so that a
  // transport thread may lag behind the forward pass.
  static constexpr uint32_t kSteps = 8;
  struct Step {
    uint64_t id = 0;
    std::vector<uint32_t> target;
    int error = KVT_OK;
    std::string message;
  };
  std::mutex mu;
  std::condition_variable cv;
  Step steps[kSteps];
  uint64_t cur_step = 0;                 // id of the newest step, 0 = none yet
  std::vector<uint32_t> submitted;       // packs of layer l handed to the GPU so far
  std::vector<uint8_t> in_graph;         // layer l's pack was recorded into a stream capture
  bool closing = false;
  uint32_t waiters = 0;

  Step& step_slot(uint64_t id) { return steps[id % kSteps]; }
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

// ----------------------------------------------------------------- session

namespace {

// One lane per layer: the layer's completion count, bumped in device memory and mirrored to
// the host. The pack kernel in front of it on the stream has ended, so its stores have left
// the caches.
// The count after `c`: 1, 2, ... 2^32 - 1, 1, ... Zero is left out on both sides (the host's
// `submitted` and the device's counter step alike), because a step's target of 0 means "not
// submitted yet".
__host__ __device__ inline uint32_t next_count(uint32_t c) { return c + 1u != 0u ? c + 1u : 1u; }

__global__ void publish_layers_kernel(uint32_t* count_dev, uint32_t* count_host, uint32_t n) {
  for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) {
    const uint32_t c = next_count(count_dev[i]);
    count_dev[i] = c;
    __hip_atomic_store(count_host + i, c, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

// Starts a new step under s->mu. Layers whose pack lives in a captured graph are counted as
// submitted now: the caller launches that graph next.
uint64_t begin_step_locked(kvt_session* s) {
  const uint64_t id = ++s->cur_step;
  kvt_session::Step& st = s->step_slot(id);
  st.id = id;
  st.error = KVT_OK;
  st.message.clear();
  st.target.assign(s->cache->n_layers, 0);
  for (uint32_t l = 0; l < s->cache->n_layers; ++l)
    if (s->in_graph[l]) st.target[l] = s->submitted[l] = next_count(s->submitted[l]);
  return id;
}

using Clock = std::chrono::steady_clock;

int timed_out(uint32_t layer) {
  return fail(KVT_ERR_TIMEOUT, "kvt_session_wait_layer_for: layer " + std::to_string(layer) +
                                   " was not complete within the time given");
}

// Blocks until completion `target` of `layer` has been published, the session is being
// destroyed, or `deadline` (if any) has passed.
int poll_layer(kvt_session* s, uint32_t layer, uint32_t target, const Clock::time_point* deadline) {
  const uint32_t* word = s->count_host + layer;
  for (uint32_t spins = 0;; ++spins) {
    // counts only grow (next_count); the comparison survives wrap-around of the 32-bit counter
    if (static_cast<int32_t>(__atomic_load_n(word, __ATOMIC_ACQUIRE) - target) >= 0) return KVT_OK;
    if (spins < 2000) {
#if defined(__x86_64__)
      __builtin_ia32_pause();
#endif
      continue;
    }
    if ((spins & 63u) == 0) {
      std::lock_guard<std::mutex> lock(s->mu);
      if (s->closing) return fail(KVT_ERR_INVALID, "kvt_session_wait_layer: the session is being destroyed");
    }
    if (deadline && Clock::now() >= *deadline) return timed_out(layer);
    if (spins < 20000)
      std::this_thread::yield();
    else
      std::this_thread::sleep_for(std::chrono::microseconds(50));
  }
}

}  // namespace

extern "C" {

int kvt_session_create(const kvt_plan* plan, const kvt_cache* cache, void* packed,
                       uint64_t layer_stride, kvt_session** out) {
  return guarded([&]() -> int {
    if (!plan || !cache || !packed || !out)
      return fail(KVT_ERR_INVALID, "kvt_session_create: null argument");
    if (layer_stride < plan->min_layer_stride)
      return fail(KVT_ERR_INVALID, "kvt_session_create: layer_stride smaller than one packed layer");
    if (int rc = check_device(plan->device)) return rc;
    DeviceGuard g;
    if (int rc = g.enter(plan->device)) return rc;
    if (int rc = kvt_plan_ready(plan)) return rc;  // save_layer may run inside a stream capture
    // destroyed through kvt_session_destroy on any early return: stream and events included
    std::unique_ptr<kvt_session, void (*)(kvt_session*)> s(new kvt_session(), kvt_session_destroy);
    s->plan = plan;
    s->cache = cache;
    s->packed = packed;
    s->layer_stride = layer_stride;
    const uint32_t n = cache->n_layers;
    KVT_HIP(hipStreamCreateWithFlags(&s->side, hipStreamNonBlocking));
    s->ready.resize(n);
    s->submitted.assign(n, 0);
    s->in_graph.assign(n, 0);
    for (uint32_t l = 0; l < n; ++l) {
      KVT_HIP(hipEventCreateWithFlags(&s->ready[l], hipEventDisableTiming));
    }
    KVT_HIP(hipEventCreateWithFlags(&s->joined, hipEventDisableTiming));
    KVT_HIP(hipEventCreateWithFlags(&s->inline_done, hipEventDisableTiming));
    KVT_HIP(hipMalloc(reinterpret_cast<void**>(&s->count_dev), n * sizeof(uint32_t)));
    KVT_HIP(hipMemset(s->count_dev, 0, n * sizeof(uint32_t)));
    KVT_HIP(hipHostMalloc(reinterpret_cast<void**>(&s->count_host), n * sizeof(uint32_t),
                          hipHostMallocCoherent));
    std::memset(s->count_host, 0, n * sizeof(uint32_t));
    *out = s.release();
    return KVT_OK;
  });
}

void kvt_session_destroy(kvt_session* s) {
  if (!s) return;
  {  // threads parked in wait_layer return with an error first
    std::unique_lock<std::mutex> lock(s->mu);
    s->closing = true;
    s->cv.notify_all();
    s->cv.wait(lock, [&] { return s->waiters == 0; });
  }
  if (s->side) {
    (void)hipStreamSynchronize(s->side);
    (void)hipStreamDestroy(s->side);
  }
  if (s->inline_any) (void)hipEventSynchronize(s->inline_done);  // packs on the caller's own stream
  if (s->inline_done) (void)hipEventDestroy(s->inline_done);
  for (hipEvent_t e : s->ready)
    if (e) (void)hipEventDestroy(e);
  if (s->joined) (void)hipEventDestroy(s->joined);
  if (s->count_dev) (void)hipFree(s->count_dev);
  if (s->count_host) (void)hipHostFree(s->count_host);
  delete s;
}

int kvt_session_set_plan(kvt_session* s, const kvt_plan* plan, void* packed, uint64_t layer_stride) {
  return guarded([&]() -> int {
    if (!s || !plan || !packed) return fail(KVT_ERR_INVALID, "kvt_session_set_plan: null argument");
    if (plan->device != s->cache->device || plan->n_tensors != s->cache->n_tensors)
      return fail(KVT_ERR_INVALID, "kvt_session_set_plan: the plan does not fit the session's cache");
    if (layer_stride < plan->min_layer_stride)
      return fail(KVT_ERR_INVALID, "kvt_session_set_plan: layer_stride smaller than one packed layer");
    std::lock_guard<std::mutex> lock(s->mu);
    // a plan slot takes its batches through kvt_plan_slot_fill: the same slot, buffer and stride
    // again change nothing a captured launch has fixed
    const bool same_slot = plan->slot && plan == s->plan && packed == s->packed && layer_stride == s->layer_stride;
    for (uint8_t g : s->in_graph)
      if (g && !same_slot)
        return fail(KVT_ERR_INVALID,
                    "kvt_session_set_plan: a captured graph still launches the session's old plan");
    s->plan = plan;
    s->packed = packed;
    s->layer_stride = layer_stride;
    return KVT_OK;
  });
}

int kvt_session_begin_step(kvt_session* s, uint64_t* step) {
  return guarded([&]() -> int {
    if (!s) return fail(KVT_ERR_INVALID, "kvt_session_begin_step: null session");
    std::lock_guard<std::mutex> lock(s->mu);
    const uint64_t id = begin_step_locked(s);
    if (step) *step = id;
    s->cv.notify_all();
    return KVT_OK;
  });
}

// The pack of layers [first, first + n) on the side stream as ONE launch, gated by `ready`
// (already recorded), and the publication of their completion.
// ready == nullptr: on `inline_stream` itself, behind whatever is queued there, with no event.
static int issue_layers(kvt_session* s, uint32_t first, uint32_t n, hipEvent_t ready,
                        hipStream_t inline_stream = nullptr) {
  auto launch = [&](bool* capturing) -> int {
    const hipStream_t on = ready ? s->side : inline_stream;
    if (ready) KVT_HIP(hipStreamWaitEvent(s->side, ready, 0));
    // a side stream that waits for an event recorded inside a capture has joined that capture
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(on, &cap) != hipSuccess) (void)hipGetLastError();
    *capturing = cap != hipStreamCaptureStatusNone;
    uint8_t* dst = static_cast<uint8_t*>(s->packed) + static_cast<uint64_t>(first) * s->layer_stride;
    if (int rc = run_plan(true, s->plan, s->cache, first, n, dst, s->layer_stride, on)) return rc;
    hipLaunchKernelGGL(publish_layers_kernel, dim3(1), dim3(64), 0, on, s->count_dev + first,
                       s->count_host + first, n);
    KVT_HIP(hipGetLastError());
    if (!ready && !*capturing) {   // kvt_session_destroy waits for it: the counters must outlive it
      KVT_HIP(hipEventRecord(s->inline_done, on));
      s->inline_any = true;
    }
    return KVT_OK;
  };
  bool capturing = false;
  const int rc = launch(&capturing);
  std::lock_guard<std::mutex> lock(s->mu);
  if (capturing) {
    // nothing runs now: the packs belong to every later launch of the graph being recorded
    if (rc == KVT_OK)
      for (uint32_t l = first; l < first + n; ++l) s->in_graph[l] = 1;
  } else {
    if (s->cur_step == 0) begin_step_locked(s);  // a session used for one step needs no begin_step
    kvt_session::Step& st = s->step_slot(s->cur_step);
    if (rc == KVT_OK) {
      for (uint32_t l = first; l < first + n; ++l)
        st.target[l] = s->submitted[l] = next_count(s->submitted[l]);
    } else if (st.error == KVT_OK) {   // latched: threads waiting for this step return it
      st.error = rc;
      st.message = kvt_last_error();
    }
  }
  if (rc == KVT_OK && ready) s->issued_any = true;   // what kvt_session_join has to wait for
  s->cv.notify_all();
  return rc;
}

static int check_layers(const kvt_session* s, uint32_t first, uint32_t n) {
  if (n == 0 || first >= s->cache->n_layers || n > s->cache->n_layers - first)
    return fail(KVT_ERR_OUT_OF_RANGE, "layer range out of range");
  return KVT_OK;
}

int kvt_session_save_layers(kvt_session* s, uint32_t first_layer, uint32_t n_layers, void* compute_stream) {
  return guarded([&]() -> int {
    if (!s) return fail(KVT_ERR_INVALID, "kvt_session_save_layers: null session");
    if (int rc = check_layers(s, first_layer, n_layers)) return rc;
    DeviceGuard g;
    if (int rc = g.enter(s->plan->device)) return rc;
    // the event of the group's last layer: everything before it on the stream has run then
    hipEvent_t ready = s->ready[first_layer + n_layers - 1];
    KVT_HIP(hipEventRecord(ready, static_cast<hipStream_t>(compute_stream)));
    return issue_layers(s, first_layer, n_layers, ready);
  });
}

int kvt_session_save_layers_inline(kvt_session* s, uint32_t first_layer, uint32_t n_layers, void* compute_stream) {
  return guarded([&]() -> int {
    if (!s) return fail(KVT_ERR_INVALID, "kvt_session_save_layers_inline: null session");
    if (int rc = check_layers(s, first_layer, n_layers)) return rc;
    DeviceGuard g;
    if (int rc = g.enter(s->plan->device)) return rc;
    return issue_layers(s, first_layer, n_layers, nullptr, static_cast<hipStream_t>(compute_stream));
  });
}

int kvt_session_save_layer(kvt_session* s, uint32_t layer, void* compute_stream) {
  return kvt_session_save_layers(s, layer, 1, compute_stream);
}

int kvt_session_save_layer_event(kvt_session* s, uint32_t layer, void* ready_event) {
  return guarded([&]() -> int {
    if (!s || !ready_event)
      return fail(KVT_ERR_INVALID, "kvt_session_save_layer_event: null argument");
    if (int rc = check_layers(s, layer, 1)) return rc;
    DeviceGuard g;
    if (int rc = g.enter(s->plan->device)) return rc;
    return issue_layers(s, layer, 1, static_cast<hipEvent_t>(ready_event));
  });
}

// deadline = nullptr: no limit.
static int wait_layer(kvt_session* s, uint64_t step, uint32_t layer, const Clock::time_point* deadline) {
  {
    if (!s) return fail(KVT_ERR_INVALID, "kvt_session_wait_layer: null session");
    if (layer >= s->cache->n_layers) return fail(KVT_ERR_OUT_OF_RANGE, "layer out of range");
    // kvt_session_destroy waits until every thread has left this function
    struct Visit {
      kvt_session* s;
      explicit Visit(kvt_session* session) : s(session) {
        std::lock_guard<std::mutex> lock(s->mu);
        ++s->waiters;
      }
      ~Visit() {
        std::lock_guard<std::mutex> lock(s->mu);
        --s->waiters;
        s->cv.notify_all();
      }
    } visit(s);
    uint32_t target = 0;
    {
      std::unique_lock<std::mutex> lock(s->mu);
      if (step == 0) step = s->cur_step ? s->cur_step : 1;  // "the current step"
      int rc = KVT_OK;
      auto settled = [&] {
        if (s->closing) {
          rc = fail(KVT_ERR_INVALID, "kvt_session_wait_layer: the session is being destroyed");
          return true;
        }
        if (s->cur_step < step) return false;                 // the step has not begun yet
        if (s->cur_step >= step + kvt_session::kSteps) {
          rc = fail(KVT_ERR_INVALID, "kvt_session_wait_layer: step " + std::to_string(step) +
                                         " is no longer tracked (the forward pass is " +
                                         std::to_string(s->cur_step - step) + " steps ahead)");
          return true;
        }
        const kvt_session::Step& st = s->step_slot(step);
        if (st.error != KVT_OK) {
          rc = fail(st.error, "kvt_session_wait_layer: the step failed: " + st.message);
          return true;
        }
        target = st.target[layer];
        return target != 0;
      };
      if (!deadline)
        s->cv.wait(lock, settled);
      else if (!s->cv.wait_until(lock, *deadline, settled))
        return timed_out(layer);
      if (rc != KVT_OK) return rc;
    }
    return poll_layer(s, layer, target, deadline);
  }
}

int kvt_session_wait_layer_step(kvt_session* s, uint64_t step, uint32_t layer) {
  return guarded([&]() -> int { return wait_layer(s, step, layer, nullptr); });
}

int kvt_session_wait_layer_for(kvt_session* s, uint64_t step, uint32_t layer, uint64_t timeout_us) {
  return guarded([&]() -> int {
    // far enough for any caller, near enough for the clock's range
    const uint64_t us = std::min<uint64_t>(timeout_us, 1000ull * 1000 * 86400 * 365);
    const Clock::time_point deadline = Clock::now() + std::chrono::microseconds(us);
    return wait_layer(s, step, layer, &deadline);
  });
}

int kvt_session_wait_layer(kvt_session* s, uint32_t layer) {
  return kvt_session_wait_layer_step(s, 0, layer);
}

int kvt_session_join(kvt_session* s, void* stream) {
  return guarded([&]() -> int {
    if (!s) return fail(KVT_ERR_INVALID, "kvt_session_join: null session");
    {
      std::lock_guard<std::mutex> lock(s->mu);
      if (!s->issued_any) return KVT_OK;
    }
    DeviceGuard g;
    if (int rc = g.enter(s->plan->device)) return rc;
    KVT_HIP(hipEventRecord(s->joined, s->side));
    KVT_HIP(hipStreamWaitEvent(static_cast<hipStream_t>(stream), s->joined, 0));
    return KVT_OK;
  });
}

void* kvt_session_side_stream(kvt_session* s) { return s ? s->side : nullptr; }

// ------------------------------------------------------------------ stager

namespace {
// The copy streams of a device's stagers: four, made together when the first stager is made and
// kept until the process ends, handed to the stagers in turn. The runtime maps streams onto a
// few hardware queues, and two streams on one queue take turns (a wait parked in the queue holds
// up everything behind it): a saving and a loading stager whose copy streams had landed on one
// queue moved 29 + 28 GB/s instead of 49 + 49. Streams made one right after the other come
// from different queues, so stagers made one after the other copy through different queues
// whatever else the process has made in between. More than four stagers share streams in turn.
constexpr int kCopyStreams = 4, kStagerDevices = 64;
struct CopyStreams {
  hipStream_t st[kCopyStreams] = {nullptr, nullptr, nullptr, nullptr};
  uint32_t next = 0;
};
std::mutex g_copy_streams_mu;
CopyStreams g_copy_streams[kStagerDevices];

// With `device` current.
int take_copy_stream(int device, hipStream_t* out) {
  if (device < 0 || device >= kStagerDevices)
    return fail(KVT_ERR_INVALID, "kvt_stager_create: device index too large");
  std::lock_guard<std::mutex> lock(g_copy_streams_mu);
  CopyStreams& c = g_copy_streams[device];
  if (!c.st[0]) {
    hipStream_t made[kCopyStreams] = {nullptr, nullptr, nullptr, nullptr};
    for (int i = 0; i < kCopyStreams; ++i) {
      const hipError_t e = hipStreamCreateWithFlags(&made[i], hipStreamNonBlocking);
      if (e != hipSuccess) {
        for (int j = 0; j < i; ++j) (void)hipStreamDestroy(made[j]);
        return hip_fail(e, "kvt_stager_create: hipStreamCreateWithFlags");
      }
    }
    for (int i = 0; i < kCopyStreams; ++i) c.st[i] = made[i];
  }
  *out = c.st[c.next++ % kCopyStreams];
  return KVT_OK;
}
}  // namespace

int kvt_stager_create(int device, uint64_t slot_bytes, uint32_t n_slots, kvt_stager** out) {
  return guarded([&]() -> int {
    if (!out || slot_bytes == 0 || n_slots < 2)
      return fail(KVT_ERR_INVALID, "kvt_stager_create: need >= 2 slots of > 0 bytes");
    if (int rc = check_device(device)) return rc;
    DeviceGuard g;
    if (int rc = g.enter(device)) return rc;
    std::unique_ptr<kvt_stager, void (*)(kvt_stager*)> s(new kvt_stager(), kvt_stager_destroy);
    s->device = device;
    s->slot_bytes = round_up(slot_bytes, 4096);
    s->n_slots = n_slots;
    KVT_HIP(hipHostMalloc(reinterpret_cast<void**>(&s->pinned), s->slot_bytes * n_slots,
                          hipHostMallocDefault));
    if (int rc = take_copy_stream(device, &s->copy)) return rc;
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
  // (the copy stream belongs to the device's set and stays; the slots' events mark this
  // stager's last copies on it)
  for (hipEvent_t e : s->slot_done)
    if (e) {
      (void)hipEventSynchronize(e);
      (void)hipEventDestroy(e);
    }
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
    if (int rc = check_device_span(dev, bytes, "kvt_stager_save: the device buffer")) return rc;
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
    if (int rc = check_device_span(dev, bytes, "kvt_stager_load: the device buffer")) return rc;
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

int kvt_measure_pcie_both_ways(int device, uint64_t bytes, uint32_t repeats, double* d2h_bytes_per_s,
                               double* h2d_bytes_per_s) {
  return guarded([&]() -> int {
    if (!d2h_bytes_per_s || !h2d_bytes_per_s || bytes == 0 || repeats == 0)
      return fail(KVT_ERR_INVALID, "kvt_measure_pcie_both_ways: bad argument");
    if (int rc = check_device(device)) return rc;
    DeviceGuard g;
    if (int rc = g.enter(device)) return rc;
    // [0] device -> host, [1] host -> device: a buffer pair and two events each. Which two streams
    // carry the copies matters (streams share a few hardware queues, and the rate of two
    // concurrent copies differs with the queues they come from), so four streams are made and
    // four pairs of them are measured; the best pair is the ceiling.
    constexpr int kStreams = 4;
    void *host[2] = {nullptr, nullptr}, *dev[2] = {nullptr, nullptr};
    hipStream_t pool[kStreams] = {nullptr, nullptr, nullptr, nullptr};
    hipEvent_t a[2] = {nullptr, nullptr}, b[2] = {nullptr, nullptr}, go = nullptr;
    int rc = KVT_OK;
    auto cleanup = [&]() {
      for (hipStream_t st : pool)
        if (st) (void)hipStreamSynchronize(st);
      for (int d = 0; d < 2; ++d) {
        if (a[d]) (void)hipEventDestroy(a[d]);
        if (b[d]) (void)hipEventDestroy(b[d]);
        if (dev[d]) (void)hipFree(dev[d]);
        if (host[d]) (void)hipHostFree(host[d]);
      }
      for (hipStream_t st : pool)
        if (st) (void)hipStreamDestroy(st);
      if (go) (void)hipEventDestroy(go);
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
    for (int d = 0; d < 2; ++d) {
      KVT_TRY(hipHostMalloc(&host[d], bytes, hipHostMallocDefault));
      KVT_TRY(hipMalloc(&dev[d], bytes));
      std::memset(host[d], 0x5a, bytes);
      KVT_TRY(hipEventCreate(&a[d]));
      KVT_TRY(hipEventCreate(&b[d]));
    }
    for (hipStream_t& st : pool) KVT_TRY(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
    KVT_TRY(hipEventCreateWithFlags(&go, hipEventDisableTiming));
    const int pairs[4][2] = {{0, 1}, {2, 3}, {0, 2}, {1, 3}};
    double best[2] = {0, 0};
    for (const auto& pr : pairs) {
      hipStream_t st[2] = {pool[pr[0]], pool[pr[1]]};
      auto copy = [&](int d) {
        return d == 0 ? hipMemcpyAsync(host[0], dev[0], bytes, hipMemcpyDeviceToHost, st[0])
                      : hipMemcpyAsync(dev[1], host[1], bytes, hipMemcpyHostToDevice, st[1]);
      };
      for (int d = 0; d < 2; ++d) KVT_TRY(copy(d));   // warm-up, both at once as well
      // both streams start their timed copies together: the second waits for the first's warm-up
      KVT_TRY(hipEventRecord(go, st[0]));
      KVT_TRY(hipStreamWaitEvent(st[1], go, 0));
      for (int d = 0; d < 2; ++d) KVT_TRY(hipEventRecord(a[d], st[d]));
      for (uint32_t i = 0; i < repeats; ++i)          // issued alternately, so that neither runs ahead
        for (int d = 0; d < 2; ++d) KVT_TRY(copy(d));
      for (int d = 0; d < 2; ++d) KVT_TRY(hipEventRecord(b[d], st[d]));
      float ms[2] = {0, 0};
      for (int d = 0; d < 2; ++d) {
        KVT_TRY(hipEventSynchronize(b[d]));
        KVT_TRY(hipEventElapsedTime(&ms[d], a[d], b[d]));
      }
      const double rate[2] = {static_cast<double>(bytes) * repeats / (ms[0] * 1e-3),
                              static_cast<double>(bytes) * repeats / (ms[1] * 1e-3)};
      if (rate[0] + rate[1] > best[0] + best[1]) best[0] = rate[0], best[1] = rate[1];
    }
#undef KVT_TRY
    *d2h_bytes_per_s = best[0];
    *h2d_bytes_per_s = best[1];
    cleanup();
    forget_device_spans();
    return KVT_OK;
  });
}

}  // extern "C"
