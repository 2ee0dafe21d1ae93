// Device kernels of libkvt_hip (gfx950 / CDNA4) and their launchers.
//
// All kernels here are pure data movement: HBM-bound byte copies with 16-byte
// vector loads/stores, 256 lanes (4 wavefronts of 64) per workgroup, several
// loads in flight per lane before the first store. No LDS, no MFMA.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "kvt_device.h"

namespace kvt {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;

// Cooperative copy of `len` bytes by the whole workgroup. Fast path: both
// pointers and the length are multiples of 16.
template <int UNROLL>
__device__ __forceinline__ void wg_copy(uint8_t* __restrict__ dst, const uint8_t* __restrict__ src,
                                        uint32_t len, uint32_t tid, uint32_t nthreads) {
  const uintptr_t mis = (reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src));
  if ((mis & 15u) == 0) {
    const uint32_t nvec = len >> 4;
    const u32x4* __restrict__ s = reinterpret_cast<const u32x4*>(src);
    u32x4* __restrict__ d = reinterpret_cast<u32x4*>(dst);
    uint32_t i = tid;
    const uint32_t step = nthreads * UNROLL;
    // full tiles: UNROLL independent loads per lane, then the stores
    for (; i + (UNROLL - 1) * nthreads < nvec; i += step) {
      u32x4 r[UNROLL];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) r[u] = __builtin_nontemporal_load(s + i + u * nthreads);
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) __builtin_nontemporal_store(r[u], d + i + u * nthreads);
    }
    for (; i < nvec; i += nthreads) __builtin_nontemporal_store(__builtin_nontemporal_load(s + i), d + i);
    const uint32_t done = nvec << 4;
    for (uint32_t j = done + tid; j < len; j += nthreads) dst[j] = src[j];
  } else if ((mis & 3u) == 0) {
    const uint32_t nw = len >> 2;
    const uint32_t* __restrict__ s = reinterpret_cast<const uint32_t*>(src);
    uint32_t* __restrict__ d = reinterpret_cast<uint32_t*>(dst);
    for (uint32_t i = tid; i < nw; i += nthreads) d[i] = s[i];
    for (uint32_t j = (nw << 2) + tid; j < len; j += nthreads) dst[j] = src[j];
  } else {
    for (uint32_t j = tid; j < len; j += nthreads) dst[j] = src[j];
  }
}

// One workgroup per (chunk, layer). PACK: cache -> packed; otherwise packed -> cache.
template <bool PACK, int UNROLL>
__global__ __launch_bounds__(kThreads) void copy_chunks_kernel(
    const Chunk* __restrict__ chunks, uint8_t* const* __restrict__ layer_ptrs, uint32_t n_tensors,
    uint32_t first_layer, uint8_t* __restrict__ packed, uint64_t layer_stride) {
  const Chunk c = chunks[blockIdx.x];
  const uint32_t layer = blockIdx.y;
  uint8_t* cache = layer_ptrs[static_cast<uint64_t>(first_layer + layer) * n_tensors + c.tensor];
  uint8_t* pk = packed + layer * layer_stride + c.packed;
  if (PACK)
    wg_copy<UNROLL>(pk, cache + c.cache_src, c.len, threadIdx.x, kThreads);
  else
    wg_copy<UNROLL>(cache + c.cache_dst, pk, c.len, threadIdx.x, kThreads);
}

// HND <-> NHD page transform. A chunk covers tokens [t0, t0 + len / (heads*row))
// of one K or V half page. Packed side: [token][head][row] contiguous from
// c.packed; cache side: [head][ntpb][row] from the half-page base. Work is
// indexed by 16-byte vector of the packed side; a row is vrow vectors.
template <bool PACK>
__global__ __launch_bounds__(kThreads) void xform_chunks_kernel(
    const Chunk* __restrict__ chunks, uint8_t* const* __restrict__ layer_ptrs, uint32_t n_tensors,
    uint32_t first_layer, uint8_t* __restrict__ packed, uint64_t layer_stride, XformDev x) {
  const Chunk c = chunks[blockIdx.x];
  const uint32_t layer = blockIdx.y;
  uint8_t* cache = layer_ptrs[static_cast<uint64_t>(first_layer + layer) * n_tensors + c.tensor] +
                   (PACK ? c.cache_src : c.cache_dst);
  uint8_t* pk = packed + layer * layer_stride + c.packed;
  const uint32_t nvec = c.len >> 4;
  u32x4* __restrict__ pv = reinterpret_cast<u32x4*>(pk);
  u32x4* __restrict__ cv = reinterpret_cast<u32x4*>(cache);
  for (uint32_t v = threadIdx.x; v < nvec; v += kThreads) {
    // exact quotients by multiply-high (operands < 2^16); a divisor of 1 has no such constant
    const uint32_t r = x.vrow == 1 ? v : __umulhi(v, x.inv_vrow);  // packed-side row: t_local*heads + h
    const uint32_t col = v - r * x.vrow;
    const uint32_t t_local = x.heads == 1 ? r : __umulhi(r, x.inv_heads);
    const uint32_t h = r - t_local * x.heads;
    const uint32_t cidx = (h * x.ntpb + c.t0 + t_local) * x.vrow + col;
    if (PACK)
      __builtin_nontemporal_store(__builtin_nontemporal_load(cv + cidx), pv + v);
    else
      __builtin_nontemporal_store(__builtin_nontemporal_load(pv + v), cv + cidx);
  }
}

// Range-granular copy driven by three int64 device arrays (the reference's
// launcher interface). blockIdx.x strides over ranges, blockIdx.y selects one
// of gridDim.y equal parts of a range (parts are multiples of 256 bytes).
__global__ __launch_bounds__(kThreads) void copy_ranges_kernel(
    const uint8_t* __restrict__ src_base, uint8_t* __restrict__ dst_base,
    const int64_t* __restrict__ src_off, const int64_t* __restrict__ dst_off,
    const int64_t* __restrict__ lens, int64_t n) {
  const uint32_t parts = gridDim.y;
  for (int64_t i = blockIdx.x; i < n; i += gridDim.x) {
    const uint64_t len = static_cast<uint64_t>(lens[i]);
    if (len == 0) continue;
    uint64_t part = (len + parts - 1) / parts;
    part = (part + 255u) & ~static_cast<uint64_t>(255u);
    const uint64_t begin = part * blockIdx.y;
    if (begin >= len) continue;
    const uint64_t end = begin + part < len ? begin + part : len;
    const uint8_t* s = src_base + src_off[i] + begin;
    uint8_t* d = dst_base + dst_off[i] + begin;
    // 32-bit inner length: walk in <= 1 GiB strides
    for (uint64_t o = 0; o < end - begin; o += (1u << 30)) {
      const uint64_t m = end - begin - o;
      wg_copy<4>(d + o, s + o, static_cast<uint32_t>(m < (1u << 30) ? m : (1u << 30)), threadIdx.x,
                 kThreads);
    }
  }
}

// Many short ranges: one wavefront (64 lanes) per range.
__global__ __launch_bounds__(kThreads) void copy_ranges_wave_kernel(
    const uint8_t* __restrict__ src_base, uint8_t* __restrict__ dst_base,
    const int64_t* __restrict__ src_off, const int64_t* __restrict__ dst_off,
    const int64_t* __restrict__ lens, int64_t n) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t waves_per_wg = kThreads / 64;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * waves_per_wg + (threadIdx.x >> 6); i < n;
       i += static_cast<int64_t>(gridDim.x) * waves_per_wg) {
    const uint64_t len = static_cast<uint64_t>(lens[i]);
    if (len == 0) continue;
    const uint8_t* s = src_base + src_off[i];
    uint8_t* d = dst_base + dst_off[i];
    for (uint64_t o = 0; o < len; o += (1u << 30)) {
      const uint64_t m = len - o;
      wg_copy<4>(d + o, s + o, static_cast<uint32_t>(m < (1u << 30) ? m : (1u << 30)), lane, 64);
    }
  }
}

// bf16 -> fp8 E4M3 (OCP "fn" variant: no infinities, 0x7F = NaN), round to
// nearest even, finite values and infinities saturate to +-448 (0x7E), NaN
// stays NaN. Integer-only so that every bit pattern is reproducible.
__device__ __forceinline__ uint32_t bf16_to_e4m3(uint32_t bits) {
  const uint32_t sign = (bits >> 8) & 0x80u;
  const uint32_t e = (bits >> 7) & 0xFFu;
  const uint32_t m = bits & 0x7Fu;
  if (e == 0xFFu) return sign | (m ? 0x7Fu : 0x7Eu);
  // below 2^-10, half of the smallest subnormal 2^-9 (the tie at 2^-10 itself goes to even = 0 below)
  if (e < 117u) return sign;
  const uint32_t sig = 0x80u | m;  // 1.mmmmmmm, value = sig * 2^(e - 134)
  const bool normal = e >= 121u;   // >= 2^-6: keep 1+3 bits; else subnormal in units of 2^-9
  const uint32_t shift = normal ? 4u : 125u - e;
  const uint32_t base = normal ? ((e - 121u) << 3) : 0u;  // exponent field minus the leading one in q
  uint32_t q = sig >> shift;
  const uint32_t rem = sig & ((1u << shift) - 1u);
  const uint32_t half = 1u << (shift - 1u);
  q += (rem > half || (rem == half && (q & 1u))) ? 1u : 0u;
  uint32_t code = base + q;
  code = code > 0x7Eu ? 0x7Eu : code;
  return sign | code;
}

__device__ __forceinline__ uint32_t cvt4(uint32_t lo, uint32_t hi) {
  return bf16_to_e4m3(lo & 0xFFFFu) | (bf16_to_e4m3(lo >> 16) << 8) |
         (bf16_to_e4m3(hi & 0xFFFFu) << 16) | (bf16_to_e4m3(hi >> 16) << 24);
}

// Converting gather: range i = lens[i] bf16 elements at src_base + src_off[i]
// -> lens[i] fp8 bytes at dst_base + dst_off[i]. Same (range, part) grid as
// copy_ranges_kernel with parts expressed in elements.
__global__ __launch_bounds__(kThreads) void convert_ranges_kernel(
    const uint8_t* __restrict__ src_base, uint8_t* __restrict__ dst_base,
    const int64_t* __restrict__ src_off, const int64_t* __restrict__ dst_off,
    const int64_t* __restrict__ lens, int64_t n) {
  const uint32_t parts = gridDim.y;
  for (int64_t i = blockIdx.x; i < n; i += gridDim.x) {
    const uint64_t count = static_cast<uint64_t>(lens[i]);
    if (count == 0) continue;
    uint64_t part = (count + parts - 1) / parts;
    part = (part + 255u) & ~static_cast<uint64_t>(255u);
    const uint64_t begin = part * blockIdx.y;
    if (begin >= count) continue;
    const uint64_t m = (begin + part < count ? begin + part : count) - begin;
    const uint8_t* s8 = src_base + src_off[i] + 2 * begin;
    uint8_t* d8 = dst_base + dst_off[i] + begin;
    const bool aligned = ((reinterpret_cast<uintptr_t>(s8) | reinterpret_cast<uintptr_t>(d8)) & 15u) == 0;
    uint64_t done = 0;
    if (aligned) {
      const uint64_t nvec = m >> 4;  // 16 elements: 32 bytes in, 16 bytes out
      const u32x4* __restrict__ s = reinterpret_cast<const u32x4*>(s8);
      u32x4* __restrict__ d = reinterpret_cast<u32x4*>(d8);
      for (uint64_t v = threadIdx.x; v < nvec; v += kThreads) {
        const u32x4 a = __builtin_nontemporal_load(s + 2 * v);
        const u32x4 b = __builtin_nontemporal_load(s + 2 * v + 1);
        u32x4 o;
        o.x = cvt4(a.x, a.y);
        o.y = cvt4(a.z, a.w);
        o.z = cvt4(b.x, b.y);
        o.w = cvt4(b.z, b.w);
        __builtin_nontemporal_store(o, d + v);
      }
      done = nvec << 4;
    }
    const uint16_t* s16 = reinterpret_cast<const uint16_t*>(s8);
    for (uint64_t j = done + threadIdx.x; j < m; j += kThreads)
      d8[j] = static_cast<uint8_t>(bf16_to_e4m3(s16[j]));
  }
}

// Plain linear copy with the gather kernel's inner loop (calibration / ceiling).
template <int UNROLL>
__global__ __launch_bounds__(kThreads) void copy_linear_kernel(uint8_t* __restrict__ dst,
                                                               const uint8_t* __restrict__ src,
                                                               uint64_t bytes, uint32_t tile) {
  const uint64_t begin = static_cast<uint64_t>(blockIdx.x) * tile;
  if (begin >= bytes) return;
  const uint64_t m = bytes - begin < tile ? bytes - begin : tile;
  wg_copy<UNROLL>(dst + begin, src + begin, static_cast<uint32_t>(m), threadIdx.x, kThreads);
}

// ----------------------------------------------------------------- launchers

hipError_t launch_copy_chunks(bool pack, const Chunk* chunks, uint32_t n_chunks,
                              uint8_t* const* layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
                              uint32_t n_layers, uint8_t* packed, uint64_t layer_stride,
                              hipStream_t stream) {
  if (n_chunks == 0 || n_layers == 0) return hipSuccess;
  const dim3 grid(n_chunks, n_layers);
  if (pack)
    hipLaunchKernelGGL((copy_chunks_kernel<true, 8>), grid, dim3(kThreads), 0, stream, chunks,
                       layer_ptrs, n_tensors, first_layer, packed, layer_stride);
  else
    hipLaunchKernelGGL((copy_chunks_kernel<false, 8>), grid, dim3(kThreads), 0, stream, chunks,
                       layer_ptrs, n_tensors, first_layer, packed, layer_stride);
  return hipGetLastError();
}

hipError_t launch_xform_chunks(bool pack, const Chunk* chunks, uint32_t n_chunks,
                               uint8_t* const* layer_ptrs, uint32_t n_tensors,
                               uint32_t first_layer, uint32_t n_layers, uint8_t* packed,
                               uint64_t layer_stride, const XformDev& x, hipStream_t stream) {
  if (n_chunks == 0 || n_layers == 0) return hipSuccess;
  const dim3 grid(n_chunks, n_layers);
  if (pack)
    hipLaunchKernelGGL((xform_chunks_kernel<true>), grid, dim3(kThreads), 0, stream, chunks,
                       layer_ptrs, n_tensors, first_layer, packed, layer_stride, x);
  else
    hipLaunchKernelGGL((xform_chunks_kernel<false>), grid, dim3(kThreads), 0, stream, chunks,
                       layer_ptrs, n_tensors, first_layer, packed, layer_stride, x);
  return hipGetLastError();
}

hipError_t launch_copy_ranges(const void* src_base, void* dst_base, const int64_t* src_off,
                              const int64_t* dst_off, const int64_t* lens, int64_t n, int num_wg,
                              int parts, bool wave_per_range, hipStream_t stream) {
  if (n <= 0) return hipSuccess;
  if (wave_per_range) {
    hipLaunchKernelGGL(copy_ranges_wave_kernel, dim3(num_wg), dim3(kThreads), 0, stream,
                       static_cast<const uint8_t*>(src_base), static_cast<uint8_t*>(dst_base),
                       src_off, dst_off, lens, n);
  } else {
    hipLaunchKernelGGL(copy_ranges_kernel, dim3(num_wg, parts), dim3(kThreads), 0, stream,
                       static_cast<const uint8_t*>(src_base), static_cast<uint8_t*>(dst_base),
                       src_off, dst_off, lens, n);
  }
  return hipGetLastError();
}

hipError_t launch_convert_ranges(const void* src_base, void* dst_base, const int64_t* src_off,
                                 const int64_t* dst_off, const int64_t* lens, int64_t n,
                                 int num_wg, int parts, hipStream_t stream) {
  if (n <= 0) return hipSuccess;
  hipLaunchKernelGGL(convert_ranges_kernel, dim3(num_wg, parts), dim3(kThreads), 0, stream,
                     static_cast<const uint8_t*>(src_base), static_cast<uint8_t*>(dst_base),
                     src_off, dst_off, lens, n);
  return hipGetLastError();
}

hipError_t launch_copy_linear(void* dst, const void* src, uint64_t bytes, hipStream_t stream) {
  if (bytes == 0) return hipSuccess;
  const uint32_t tile = 32768;
  const uint64_t wgs = (bytes + tile - 1) / tile;
  hipLaunchKernelGGL((copy_linear_kernel<8>), dim3(static_cast<uint32_t>(wgs)), dim3(kThreads), 0,
                     stream, static_cast<uint8_t*>(dst), static_cast<const uint8_t*>(src), bytes,
                     tile);
  return hipGetLastError();
}

}  // namespace kvt
