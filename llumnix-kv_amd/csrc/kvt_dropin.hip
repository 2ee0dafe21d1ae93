// The reference's copy entry points, same calling conventions: range lists as
// three int64 device arrays, or kvt_ipc_block lists with caller-owned metadata
// buffers.
#include <algorithm>
#include <atomic>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "kvt_runtime.h"

using namespace kvt;

namespace {

int range_launch_shape(int64_t n, int num_wg, int* wgs) {
  if (n > 0x7FFFFFFFll) return fail(KVT_ERR_INVALID, "too many ranges");
  int w = num_wg > 0 ? num_wg : static_cast<int>(std::min<int64_t>(n, 1 << 20));
  *wgs = std::max(1, w);
  return KVT_OK;
}

int launch_ranges(bool convert, const void* src, void* dst, const int64_t* so, const int64_t* dof,
                  const int64_t* len, int64_t n, int num_wg, int threads_per_wg, void* stream) {
  (void)threads_per_wg;  // workgroups are always 256 lanes (4 wavefronts)
  if (n == 0) return KVT_OK;
  if (n < 0 || !src || !dst || !so || !dof || !len)
    return fail(KVT_ERR_INVALID, "launch_copy: bad argument");
  if (usable_devices() <= 0) return fail(KVT_ERR_NO_DEVICE, "no usable gfx950 (MI355X) device");
  int wgs = 0;
  if (int rc = range_launch_shape(n, num_wg, &wgs)) return rc;
  // The range lengths live on the device, so the grid cannot be sized to them: `rows`
  // workgroups stride over the 4 KiB slices of each range. One slice per workgroup is the
  // fastest shape, but workgroups that find nothing to do are not free (35 000 ranges of 8
  // slices: 6.0 TB/s with 1 row, 6.3 with 2, 6.45 with 4, 6.5 with 8, 4.5 with 16, 2.2 with
  // 64), so a long list gets 2 rows (at most half idle even for one-slice ranges) and only a
  // short one more (enough to fill the device when its ranges are long).
  const int rows = static_cast<int>(std::max<int64_t>(2, std::min<int64_t>(64, (8192 + n - 1) / n)));
  const hipStream_t s = static_cast<hipStream_t>(stream);
  int device = 0;   // these entry points name no device: the caller's current one
  KVT_HIP(hipGetDevice(&device));
  const uint32_t cap = copy_wg_cap(device);
  const hipError_t e = convert ? launch_convert_ranges(src, dst, so, dof, len, n, wgs, rows, cap, s)
                               : launch_copy_ranges(src, dst, so, dof, len, n, wgs, rows, cap, s);
  if (e != hipSuccess) return hip_fail(e, "range copy launch");
  return KVT_OK;
}

// When a list goes to the DMA engines instead of a kernel (kvt_set_copy_memcpy_thresholds).
constexpr uint64_t kDmaMaxRanges = 16, kDmaMinBytes = 8ull << 20;
std::atomic<uint64_t> g_dma_max_ranges{kDmaMaxRanges}, g_dma_min_bytes{kDmaMinBytes};

// Workgroups per range when the lengths are known on the host: the mean number of slices
// per range (bounded). Equal lengths then get exactly one slice per workgroup, the fastest
// shape; in a mixed list the few long ranges are strided over by their `rows` workgroups
// instead of every short range paying for idle ones.
int rows_for(uint64_t slices, uint64_t n_ranges) {
  return static_cast<int>(std::min<uint64_t>(std::max<uint64_t>(1, (slices + n_ranges - 1) / n_ranges), 512));
}

// Shared body of the two "handle data" entry points. `halve`: converting
// gather (contiguous side advances by length / 2, lengths passed to the kernel
// are element counts).
int handle_data(void* tensor_buf, void* layer_gpu_ptr, const kvt_ipc_block* blocks, uint64_t n,
                uint64_t tensor_data_size, int direction, bool halve, int device, void* stream,
                int64_t* dev_meta, int64_t* host_meta, int64_t max_block_num) {
  if (n == 0) return KVT_OK;
  if (!tensor_buf || !layer_gpu_ptr || !blocks || !dev_meta || !host_meta)
    return fail(KVT_ERR_INVALID, "copy_handle_data: null argument");
  if (direction != KVT_COPY_H2D && direction != KVT_COPY_D2H)
    return fail(KVT_ERR_INVALID, "copy_handle_data: bad direction");
  if (int rc = check_device(device)) return rc;
  if (max_block_num <= 0) max_block_num = 8192;
  uint64_t total = 0, layer_extent = 0, shortest = ~0ull, longest = 0;
  for (uint64_t i = 0; i < n; ++i) {
    if (blocks[i].length == 0) return fail(KVT_ERR_INVALID, "copy_handle_data: zero-length range");
    if (halve && (blocks[i].length & 1)) return fail(KVT_ERR_INVALID, "odd bf16 byte length");
    total += blocks[i].length;
    shortest = std::min(shortest, blocks[i].length);
    longest = std::max(longest, blocks[i].length);
    layer_extent = std::max(layer_extent, blocks[i].dst_offset + blocks[i].length);
  }
  if (total != tensor_data_size)
    return fail(KVT_ERR_INVALID, "copy_handle_data: tensor_data_size != sum of range lengths");
  DeviceGuard g;
  if (int rc = g.enter(device)) return rc;
  if (int rc = check_device_span(tensor_buf, halve ? total / 2 : total,
                                 "copy_handle_data: the contiguous buffer"))
    return rc;
  if (int rc = check_device_span(layer_gpu_ptr, layer_extent, "copy_handle_data: the layer tensor"))
    return rc;
  const hipStream_t s = static_cast<hipStream_t>(stream);
  // A few very large ranges go to the DMA engines, one copy each. The reference makes this
  // choice (memcpy loop or kernel) from a profile it takes at start-up
  // (copy_kernels.cpp:495-619); here it is fixed from measurements on MI355X: against pinned
  // host memory a copy of 128 MiB runs at 57 GB/s where the kernel's stores across PCIe reach
  // 54, the kernel wins below about 8 MiB per copy (2 MiB: 53 against 33 GB/s).
  if (!halve && n <= g_dma_max_ranges.load(std::memory_order_relaxed) &&
      shortest >= g_dma_min_bytes.load(std::memory_order_relaxed)) {
    uint64_t cursor = 0;
    for (uint64_t i = 0; i < n; ++i) {
      uint8_t* host = static_cast<uint8_t*>(tensor_buf) + cursor;
      uint8_t* dev = static_cast<uint8_t*>(layer_gpu_ptr) + blocks[i].dst_offset;
      if (direction == KVT_COPY_D2H)
        KVT_HIP(hipMemcpyAsync(host, dev, blocks[i].length, hipMemcpyDefault, s));
      else
        KVT_HIP(hipMemcpyAsync(dev, host, blocks[i].length, hipMemcpyDefault, s));
      cursor += blocks[i].length;
    }
    return KVT_OK;
  }
  // What the kernel has to move: {position in the contiguous buffer, cache offset, length}.
  // In a list of mixed lengths the ranges long enough for a DMA copy go there one by one and
  // only the rest to the kernel (the reference's enqueue_hybrid_copy, copy_kernels.cpp:675-722,
  // with its per-range rule select_single_block_method, :621-631).
  static thread_local std::vector<kvt_ipc_block> work;
  work.clear();
  const uint64_t dma_min = g_dma_min_bytes.load(std::memory_order_relaxed);
  const bool split = !halve && shortest != longest && longest >= dma_min &&
                     g_dma_max_ranges.load(std::memory_order_relaxed) != 0;
  {
    uint64_t cursor = 0;
    for (uint64_t i = 0; i < n; ++i) {
      const kvt_ipc_block& b = blocks[i];
      if (split && b.length >= dma_min) {
        uint8_t* host = static_cast<uint8_t*>(tensor_buf) + cursor;
        uint8_t* dev = static_cast<uint8_t*>(layer_gpu_ptr) + b.dst_offset;
        if (direction == KVT_COPY_D2H)
          KVT_HIP(hipMemcpyAsync(host, dev, b.length, hipMemcpyDefault, s));
        else
          KVT_HIP(hipMemcpyAsync(dev, host, b.length, hipMemcpyDefault, s));
      } else {
        work.push_back(kvt_ipc_block{cursor, b.dst_offset, b.length});
      }
      cursor += halve ? b.length / 2 : b.length;
    }
  }
  const uint64_t n_work = work.size();
  for (uint64_t first = 0; first < n_work; first += static_cast<uint64_t>(max_block_num)) {
    const uint64_t m = std::min<uint64_t>(static_cast<uint64_t>(max_block_num), n_work - first);
    int64_t* contig = host_meta;
    int64_t* gpu = host_meta + m;
    int64_t* lens = host_meta + 2 * m;
    const uint64_t unit = halve ? 8192 : 4096;  // source bytes of one workgroup's slice
    uint64_t slices = 0;
    for (uint64_t i = 0; i < m; ++i) {
      const kvt_ipc_block& b = work[first + i];
      contig[i] = static_cast<int64_t>(b.src_offset);
      gpu[i] = static_cast<int64_t>(b.dst_offset);
      lens[i] = static_cast<int64_t>(halve ? b.length / 2 : b.length);
      slices += (b.length + unit - 1) / unit;
    }
    KVT_HIP(hipMemcpyAsync(dev_meta, host_meta, 3 * m * sizeof(int64_t), hipMemcpyHostToDevice, s));
    const int64_t* d_contig = dev_meta;
    const int64_t* d_gpu = dev_meta + m;
    const int64_t* d_lens = dev_meta + 2 * m;
    const int wgs = static_cast<int>(m);
    const int rows = rows_for(slices, m);
    const uint32_t cap = copy_wg_cap(device);
    hipError_t e;
    if (halve)
      e = launch_convert_ranges(layer_gpu_ptr, tensor_buf, d_gpu, d_contig, d_lens,
                                static_cast<int64_t>(m), wgs, rows, cap, s);
    else if (direction == KVT_COPY_D2H)
      e = launch_copy_ranges(layer_gpu_ptr, tensor_buf, d_gpu, d_contig, d_lens,
                             static_cast<int64_t>(m), wgs, rows, cap, s);
    else
      e = launch_copy_ranges(tensor_buf, layer_gpu_ptr, d_contig, d_gpu, d_lens,
                             static_cast<int64_t>(m), wgs, rows, cap, s);
    if (e != hipSuccess) return hip_fail(e, "copy_handle_data launch");
    // the metadata buffers are reused by the next batch
    if (first + m < n_work) KVT_HIP(hipStreamSynchronize(s));
  }
  return KVT_OK;
}

// Single batch with separate device arrays (copy_handle_data_kernel_direct).
// meta_by_kernel: the three device arrays are one piece of 3 n int64 starting at src_dev, and
// the metadata reaches it through a copy kernel reading host_meta (device-visible pinned
// memory) instead of three runtime copies.
int handle_data_direct(void* tensor_buf, void* layer_gpu_ptr, const kvt_ipc_block* blocks,
                       uint64_t n, uint64_t tensor_data_size, int direction, int device,
                       void* stream, int64_t* src_dev, int64_t* dst_dev, int64_t* len_dev,
                       int64_t* host_meta, bool explicit_host_offsets, bool meta_by_kernel = false) {
  if (n == 0) return KVT_OK;
  if (!tensor_buf || !layer_gpu_ptr || !blocks || !src_dev || !dst_dev || !len_dev || !host_meta)
    return fail(KVT_ERR_INVALID, "copy_handle_data_kernel_direct: null argument");
  if (direction != KVT_COPY_H2D && direction != KVT_COPY_D2H)
    return fail(KVT_ERR_INVALID, "copy_handle_data_kernel_direct: bad direction");
  if (n > 0x7FFFFFFFull) return fail(KVT_ERR_INVALID, "too many ranges");
  if (int rc = check_device(device)) return rc;
  uint64_t cursor = 0, slices = 0, layer_extent = 0;
  for (uint64_t i = 0; i < n; ++i) {
    const kvt_ipc_block& b = blocks[i];
    layer_extent = std::max(layer_extent, b.dst_offset + b.length);
    const uint64_t host_off = explicit_host_offsets ? b.src_offset : cursor;
    if (b.length == 0 || host_off > tensor_data_size || b.length > tensor_data_size - host_off)
      return fail(KVT_ERR_OUT_OF_RANGE,
                  "copy_handle_data_kernel_direct: range outside the contiguous buffer");
    host_meta[i] = static_cast<int64_t>(host_off);
    host_meta[n + i] = static_cast<int64_t>(b.dst_offset);
    host_meta[2 * n + i] = static_cast<int64_t>(b.length);
    cursor += b.length;
    slices += (b.length + 4095) / 4096;
  }
  if (!explicit_host_offsets && cursor != tensor_data_size)
    return fail(KVT_ERR_INVALID,
                "copy_handle_data_kernel_direct: tensor_data_size != sum of range lengths");
  DeviceGuard g;
  if (int rc = g.enter(device)) return rc;
  if (int rc = check_device_span(tensor_buf, tensor_data_size,
                                 "copy_handle_data_kernel_direct: the contiguous buffer"))
    return rc;
  if (int rc = check_device_span(layer_gpu_ptr, layer_extent,
                                 "copy_handle_data_kernel_direct: the layer tensor"))
    return rc;
  const hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t bytes = n * sizeof(int64_t);
  if (meta_by_kernel) {
    if (int rc = check_device_span(host_meta, 3 * bytes,
                                   "copy_handle_data_kernel_direct: the metadata staging buffer"))
      return rc;
    const hipError_t me = launch_copy_linear(src_dev, host_meta, 3 * bytes, s);
    if (me != hipSuccess) return hip_fail(me, "metadata copy launch");
  } else {
    KVT_HIP(hipMemcpyAsync(src_dev, host_meta, bytes, hipMemcpyHostToDevice, s));
    KVT_HIP(hipMemcpyAsync(dst_dev, host_meta + n, bytes, hipMemcpyHostToDevice, s));
    KVT_HIP(hipMemcpyAsync(len_dev, host_meta + 2 * n, bytes, hipMemcpyHostToDevice, s));
  }
  const int rows = rows_for(slices, n);
  const hipError_t e =
      direction == KVT_COPY_D2H
          ? launch_copy_ranges(layer_gpu_ptr, tensor_buf, dst_dev, src_dev, len_dev,
                               static_cast<int64_t>(n), static_cast<int>(n), rows, copy_wg_cap(device), s)
          : launch_copy_ranges(tensor_buf, layer_gpu_ptr, src_dev, dst_dev, len_dev,
                               static_cast<int64_t>(n), static_cast<int>(n), rows, copy_wg_cap(device), s);
  if (e != hipSuccess) return hip_fail(e, "copy_handle_data_kernel_direct launch");
  return KVT_OK;
}

}  // namespace

extern "C" {

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

int kvt_launch_copy_int64_array_h2d(const int64_t* host_src, int64_t* device_dst,
                                    int64_t num_elements, int num_wg, int threads_per_wg,
                                    void* stream) {
  (void)num_wg;          // one 256-lane workgroup per 4 KiB, like every other copy here
  (void)threads_per_wg;
  return guarded([&]() -> int {
    if (num_elements == 0) return KVT_OK;
    if (num_elements < 0 || !host_src || !device_dst)
      return fail(KVT_ERR_INVALID, "launch_copy_int64_array_h2d: bad argument");
    if (usable_devices() <= 0) return fail(KVT_ERR_NO_DEVICE, "no usable gfx950 (MI355X) device");
    if (num_elements > (1ll << 40)) return fail(KVT_ERR_INVALID, "launch_copy_int64_array_h2d: too large");
    const uint64_t bytes = static_cast<uint64_t>(num_elements) * sizeof(int64_t);
    // both sides must be memory a kernel can touch: the source is pinned host memory
    if (int rc = check_device_span(host_src, bytes, "launch_copy_int64_array_h2d: the host array")) return rc;
    if (int rc = check_device_span(device_dst, bytes, "launch_copy_int64_array_h2d: the device array"))
      return rc;
    const hipError_t e = launch_copy_linear(device_dst, host_src, bytes, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "int64 array copy launch");
    return KVT_OK;
  });
}

// Per-thread metadata buffers and streams of the copy threads (CopyKernelCtx,
// kvtransfer/src/copy_utils.cpp:9-154): created on first use, re-created when the thread
// moves to another device or asks for more ranges, released when the thread ends.
namespace {
struct CopyThreadCtx {
  int device = -1;
  int64_t capacity = 0;  // ranges
  int64_t* dev = nullptr;
  int64_t* host = nullptr;
  hipStream_t streams[2] = {nullptr, nullptr};  // KVT_COPY_H2D, KVT_COPY_D2H

  void release() {
    if (device >= 0) (void)hipSetDevice(device);
    for (hipStream_t& st : streams)
      if (st) {
        (void)hipStreamSynchronize(st);  // the streams may still reference the buffers
        (void)hipStreamDestroy(st);
        st = nullptr;
      }
    if (dev) (void)hipFree(dev);
    if (host) (void)hipHostFree(host);
    dev = host = nullptr;
    capacity = 0;
  }
  ~CopyThreadCtx() { release(); }
};
thread_local CopyThreadCtx g_copy_ctx;
}  // namespace

int kvt_get_kernel_copy_buffer(int device, int64_t max_block_num, int64_t** dev_meta,
                               int64_t** host_meta) {
  return guarded([&]() -> int {
    if (!dev_meta || !host_meta)
      return fail(KVT_ERR_INVALID, "kvt_get_kernel_copy_buffer: null argument");
    if (int rc = check_device(device)) return rc;
    if (max_block_num <= 0) max_block_num = 8192;
    CopyThreadCtx& c = g_copy_ctx;
    if (c.device != device || c.capacity < max_block_num) {
      DeviceGuard g;
      if (int rc = g.enter(device)) return rc;
      c.release();
      c.device = device;
      const size_t bytes = 3 * sizeof(int64_t) * static_cast<size_t>(max_block_num);
      KVT_HIP(hipMalloc(reinterpret_cast<void**>(&c.dev), bytes));
      const hipError_t e = hipHostMalloc(reinterpret_cast<void**>(&c.host), bytes, hipHostMallocDefault);
      if (e != hipSuccess) {
        c.release();
        return hip_fail(e, "kvt_get_kernel_copy_buffer: pinned metadata buffer");
      }
      c.capacity = max_block_num;
    }
    *dev_meta = c.dev;
    *host_meta = c.host;
    return KVT_OK;
  });
}

int kvt_get_thread_local_stream(int device, int direction, void** stream) {
  return guarded([&]() -> int {
    if (!stream || (direction != KVT_COPY_H2D && direction != KVT_COPY_D2H))
      return fail(KVT_ERR_INVALID, "kvt_get_thread_local_stream: bad argument");
    if (int rc = check_device(device)) return rc;
    CopyThreadCtx& c = g_copy_ctx;
    if (c.device != device) {
      c.release();
      c.device = device;
    }
    if (!c.streams[direction]) {
      DeviceGuard g;
      if (int rc = g.enter(device)) return rc;
      KVT_HIP(hipStreamCreateWithFlags(&c.streams[direction], hipStreamNonBlocking));
    }
    *stream = c.streams[direction];
    return KVT_OK;
  });
}

int kvt_set_copy_memcpy_thresholds(uint64_t min_range_bytes, uint64_t max_ranges) {
  if (min_range_bytes == 0)
    return fail(KVT_ERR_INVALID, "kvt_set_copy_memcpy_thresholds: min_range_bytes must be positive");
  g_dma_min_bytes.store(min_range_bytes, std::memory_order_relaxed);
  g_dma_max_ranges.store(max_ranges, std::memory_order_relaxed);
  return KVT_OK;
}

int kvt_get_copy_memcpy_thresholds(uint64_t* min_range_bytes, uint64_t* max_ranges) {
  if (min_range_bytes) *min_range_bytes = g_dma_min_bytes.load(std::memory_order_relaxed);
  if (max_ranges) *max_ranges = g_dma_max_ranges.load(std::memory_order_relaxed);
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

int kvt_copy_handle_data_kernel_direct(void* tensor_buf, void* layer_gpu_ptr,
                                       const kvt_ipc_block* blocks, uint64_t n,
                                       uint64_t tensor_data_size, int direction, int device,
                                       void* stream, int64_t* src_offsets_dev,
                                       int64_t* dst_offsets_dev, int64_t* lengths_dev,
                                       int64_t* host_meta, int use_explicit_host_offsets) {
  return guarded([&]() {
    return handle_data_direct(tensor_buf, layer_gpu_ptr, blocks, n, tensor_data_size, direction,
                              device, stream, src_offsets_dev, dst_offsets_dev, lengths_dev,
                              host_meta, use_explicit_host_offsets != 0);
  });
}

// ------------------------------------------------ the entry point that allocates nothing

}  // extern "C"

// Device-side range metadata of kvt_copy_handle_data_kernel_direct_static: three int64 arrays
// of up to kStaticMaxRanges entries, 192 KiB, held by every GPU the library runs on until the
// process ends. In host code the name is only a handle for hipGetSymbolAddress; each device
// has its own copy at its own address, looked up once per device (g_scratch_ptr).
constexpr uint64_t kStaticMaxRanges = 8192;
static __device__ __align__(256) int64_t scratch[3 * kStaticMaxRanges];

namespace {
constexpr int kMaxStaticDevices = 64;
std::mutex g_scratch_mu;
int64_t* g_scratch_ptr[kMaxStaticDevices] = {};

// The address of `device`'s copy of the array (looked up with that device current).
int static_scratch(int device, int64_t** out) {
  if (device < 0 || device >= kMaxStaticDevices)
    return fail(KVT_ERR_INVALID, "device index too large for the static metadata array");
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[device]) {
    DeviceGuard g;
    if (int rc = g.enter(device)) return rc;
    void* p = nullptr;
    KVT_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return fail(KVT_ERR_HIP, "hipGetSymbolAddress gave no address for the static metadata array");
    g_scratch_ptr[device] = static_cast<int64_t*>(p);
  }
  *out = g_scratch_ptr[device];
  return KVT_OK;
}
}  // namespace

extern "C" {

int kvt_initialize_copy_method_profile(int device) {
  return guarded([&]() -> int {
    if (int rc = check_device(device)) return rc;
    int64_t* unused = nullptr;
    return static_scratch(device, &unused);
  });
}

int kvt_copy_handle_data_kernel_direct_static(void* tensor_buf, void* layer_gpu_ptr,
                                              const kvt_ipc_block* blocks, uint64_t n,
                                              uint64_t tensor_data_size, int direction, int device,
                                              void* stream, int64_t* host_meta,
                                              int use_explicit_host_offsets) {
  return guarded([&]() -> int {
    if (n > kStaticMaxRanges)
      return fail(KVT_ERR_INVALID,
                  "kvt_copy_handle_data_kernel_direct_static: at most 8192 ranges per call (" +
                      std::to_string(n) + " given)");
    if (n == 0) return KVT_OK;
    if (int rc = check_device(device)) return rc;
    int64_t* meta = nullptr;
    if (int rc = static_scratch(device, &meta)) return rc;
    return handle_data_direct(tensor_buf, layer_gpu_ptr, blocks, n, tensor_data_size, direction,
                              device, stream, meta, meta + n, meta + 2 * n, host_meta,
                              use_explicit_host_offsets != 0, true);
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

}  // extern "C"
