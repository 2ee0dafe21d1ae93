// Layer-message framing of the staged transports (host side), and the range
// lists of per-block store objects.
//
// A staged channel sends one message per layer: a small header, the range
// metadata and the packed blob(s). Writing the frame around a blob that the
// GPU packs (or a DMA engine copies) straight into the send buffer removes the
// extra host copy; parsing it on the receiving side yields the ranges and blob
// positions for the unpack.
//
//   TCP          [magic u32][reqid u64][layer u64][num_tensors u64]
//                per tensor: [n u64][n x {src,dst,len u64}][blob_bytes u64][blob]
//   staged RDMA  [magic u32][reqid u64][total_len u64][layer u64]
//                [n u64][n x {src,dst,len u64}][blob]            (one tensor only)
#include <cstring>

#include "kvt_internal.h"

namespace kvt {
namespace {

constexpr uint64_t kRpcHeader = 4 + 8;

void put64(uint8_t* p, uint64_t v) { std::memcpy(p, &v, 8); }
uint64_t get64(const uint8_t* p) {
  uint64_t v;
  std::memcpy(&v, p, 8);
  return v;
}

// Sum of the range lengths; saturates, so that lengths chosen to wrap around to a plausible
// total cannot pass for it.
uint64_t blob_bytes_of(const RunList& runs) {
  uint64_t total = 0;
  for (const kvt_ipc_block& r : runs)
    if (__builtin_add_overflow(total, r.length, &total)) return ~0ull;
  return total;
}

int layout_of(int format, const kvt_block_lists& lists, kvt_wire_layout* out) {
  std::memset(out, 0, sizeof(*out));
  const size_t nt = lists.tensors.size();
  if (nt == 0 || nt > KVT_MAX_TENSORS) return fail(KVT_ERR_INVALID, "wire: tensor count out of range");
  out->n_tensors = static_cast<uint32_t>(nt);
  uint64_t cur;
  if (format == KVT_WIRE_TCP) {
    cur = kRpcHeader + 8 + 8;
    for (size_t t = 0; t < nt; ++t) {
      out->meta_offset[t] = cur;
      cur += 8 + lists.tensors[t].size() * sizeof(kvt_ipc_block) + 8;
      out->blob_offset[t] = cur;
      out->blob_bytes[t] = blob_bytes_of(lists.tensors[t]);
      if (__builtin_add_overflow(cur, out->blob_bytes[t], &cur))
        return fail(KVT_ERR_OVERFLOW, "wire: frame size does not fit 64 bits");
    }
  } else if (format == KVT_WIRE_RDMA_STAGED) {
    if (nt != 1) return fail(KVT_ERR_INVALID, "wire: the staged RDMA frame carries one tensor per layer");
    cur = kRpcHeader + 8 + 8;
    out->meta_offset[0] = cur;
    cur += 8 + lists.tensors[0].size() * sizeof(kvt_ipc_block);
    out->blob_offset[0] = cur;
    out->blob_bytes[0] = blob_bytes_of(lists.tensors[0]);
    if (__builtin_add_overflow(cur, out->blob_bytes[0], &cur))
      return fail(KVT_ERR_OVERFLOW, "wire: frame size does not fit 64 bits");
  } else {
    return fail(KVT_ERR_INVALID, "wire: unknown frame format");
  }
  out->total_bytes = cur;
  return KVT_OK;
}

}  // namespace
}  // namespace kvt

using namespace kvt;

extern "C" {

int kvt_wire_layout_of(int format, const kvt_block_lists* lists, kvt_wire_layout* out) {
  return guarded([&]() -> int {
    if (!lists || !out) return fail(KVT_ERR_INVALID, "kvt_wire_layout_of: null argument");
    return layout_of(format, *lists, out);
  });
}

int kvt_wire_write_frame(int format, void* buf, uint64_t capacity, uint64_t reqid,
                         uint64_t layer_idx, const kvt_block_lists* lists, kvt_wire_layout* out) {
  return guarded([&]() -> int {
    if (!buf || !lists) return fail(KVT_ERR_INVALID, "kvt_wire_write_frame: null argument");
    kvt_wire_layout lay;
    if (int rc = layout_of(format, *lists, &lay)) return rc;
    if (lay.total_bytes > capacity)
      return fail(KVT_ERR_OUT_OF_RANGE, "kvt_wire_write_frame: buffer smaller than the frame");
    uint8_t* p = static_cast<uint8_t*>(buf);
    const uint32_t magic = KVT_WIRE_MAGIC;
    std::memcpy(p, &magic, 4);
    put64(p + 4, reqid);
    if (format == KVT_WIRE_TCP) {
      put64(p + kRpcHeader, layer_idx);
      put64(p + kRpcHeader + 8, lay.n_tensors);
    } else {
      put64(p + kRpcHeader, lay.total_bytes);
      put64(p + kRpcHeader + 8, layer_idx);
    }
    for (uint32_t t = 0; t < lay.n_tensors; ++t) {
      const RunList& runs = lists->tensors[t];
      uint8_t* m = p + lay.meta_offset[t];
      put64(m, runs.size());
      if (!runs.empty()) std::memcpy(m + 8, runs.data(), runs.size() * sizeof(kvt_ipc_block));
      if (format == KVT_WIRE_TCP) put64(m + 8 + runs.size() * sizeof(kvt_ipc_block), lay.blob_bytes[t]);
    }
    if (out) *out = lay;
    return KVT_OK;
  });
}

int kvt_wire_parse_frame(int format, const void* buf, uint64_t len, uint32_t expect_tensors,
                         uint64_t* reqid, uint64_t* layer_idx, kvt_block_lists* lists,
                         kvt_wire_layout* out) {
  return guarded([&]() -> int {
    if (!buf || !lists || !out) return fail(KVT_ERR_INVALID, "kvt_wire_parse_frame: null argument");
    const uint8_t* p = static_cast<const uint8_t*>(buf);
    std::memset(out, 0, sizeof(*out));
    lists->tensors.clear();
    if (format != KVT_WIRE_TCP && format != KVT_WIRE_RDMA_STAGED)
      return fail(KVT_ERR_INVALID, "wire: unknown frame format");
    const uint64_t fixed = kRpcHeader + 8 + 8 + (format == KVT_WIRE_RDMA_STAGED ? 8 : 0);
    if (len < fixed) return fail(KVT_ERR_INVALID, "wire: message too short");
    uint32_t magic;
    std::memcpy(&magic, p, 4);
    if (magic != KVT_WIRE_MAGIC) return fail(KVT_ERR_INVALID, "wire: bad magic");
    if (reqid) *reqid = get64(p + 4);
    uint64_t cur = kRpcHeader;
    if (format == KVT_WIRE_TCP) {
      if (layer_idx) *layer_idx = get64(p + cur);
      const uint64_t nt = get64(p + cur + 8);
      cur += 16;
      if (nt == 0 || nt > KVT_MAX_TENSORS || (expect_tensors && nt != expect_tensors))
        return fail(KVT_ERR_INVALID, "wire: num_tensors mismatch");
      out->n_tensors = static_cast<uint32_t>(nt);
      lists->tensors.resize(nt);
      for (uint64_t t = 0; t < nt; ++t) {
        if (len - cur < 8) return fail(KVT_ERR_INVALID, "wire: truncated at metadata_size");
        out->meta_offset[t] = cur;
        const uint64_t n = get64(p + cur);
        cur += 8;
        if (n > (len - cur) / sizeof(kvt_ipc_block) || len - cur - n * sizeof(kvt_ipc_block) < 8)
          return fail(KVT_ERR_INVALID, "wire: incomplete metadata");
        lists->tensors[t].resize(n);
        if (n) std::memcpy(lists->tensors[t].data(), p + cur, n * sizeof(kvt_ipc_block));
        cur += n * sizeof(kvt_ipc_block);
        const uint64_t bytes = get64(p + cur);
        cur += 8;
        if (bytes > len - cur) return fail(KVT_ERR_INVALID, "wire: truncated tensor data");
        out->blob_offset[t] = cur;
        out->blob_bytes[t] = bytes;
        cur += bytes;
      }
      out->total_bytes = cur;
    } else {
      const uint64_t total = get64(p + cur);
      if (total > len) return fail(KVT_ERR_INVALID, "wire: stated length exceeds the message");
      if (layer_idx) *layer_idx = get64(p + cur + 8);
      cur += 16;
      if (expect_tensors > 1) return fail(KVT_ERR_INVALID, "wire: num_tensors mismatch");
      out->n_tensors = 1;
      out->meta_offset[0] = cur;
      const uint64_t n = get64(p + cur);
      cur += 8;
      if (total < cur || n > (total - cur) / sizeof(kvt_ipc_block))
        return fail(KVT_ERR_INVALID, "wire: incomplete metadata");
      lists->tensors.resize(1);
      lists->tensors[0].resize(n);
      if (n) std::memcpy(lists->tensors[0].data(), p + cur, n * sizeof(kvt_ipc_block));
      cur += n * sizeof(kvt_ipc_block);
      out->blob_offset[0] = cur;
      out->blob_bytes[0] = total - cur;
      out->total_bytes = total;
    }
    // the blob must hold exactly the bytes the ranges describe
    for (uint32_t t = 0; t < out->n_tensors; ++t)
      if (blob_bytes_of(lists->tensors[t]) != out->blob_bytes[t])
        return fail(KVT_ERR_INVALID, "wire: blob size differs from the sum of range lengths");
    return KVT_OK;
  });
}

int kvt_block_object_lists(int cache_shape, const kvt_worker_info* src, const kvt_worker_info* dst,
                           const uint32_t* src_blocks, const uint32_t* dst_blocks, uint64_t n,
                           kvt_block_lists* lists, uint64_t* object_bytes) {
  return guarded([&]() -> int {
    if (!src || !dst || (!src_blocks && n) || (!dst_blocks && n) || !lists)
      return fail(KVT_ERR_INVALID, "kvt_block_object_lists: null argument");
    if (src->n_tensors < 1 || dst->n_tensors < 1 || src->n_tensors != dst->n_tensors)
      return fail(KVT_ERR_INVALID, "kvt_block_object_lists: tensor count mismatch");
    const uint32_t nt = src->n_tensors;
    if (lists->tensors.size() < nt) lists->tensors.resize(nt);
    uint64_t obj = 0;
    for (uint32_t t = 0; t < nt; ++t) {
      const uint64_t B = src->block_sizes[t];
      if (B != dst->block_sizes[t])
        return fail(KVT_ERR_INVALID, "kvt_block_object_lists: block sizes differ");
      obj += B;
      RunList& out = lists->tensors[t];
      const uint64_t s_cap = B * src->layer_num_blocks, d_cap = B * dst->layer_num_blocks;
      for (uint64_t i = 0; i < n; ++i) {
        if (src_blocks[i] >= src->layer_num_blocks || dst_blocks[i] >= dst->layer_num_blocks)
          return fail(KVT_ERR_OUT_OF_RANGE, "kvt_block_object_lists: block id outside the pool");
        if (cache_shape == KVT_SHAPE_FLASH) {
          // [2, nblk, bs, h, d]: the object is K block then V block (kvcache[:, blk])
          const uint64_t half = B / 2;
          out.push_back(kvt_ipc_block{src_blocks[i] * half, dst_blocks[i] * half, half});
          out.push_back(kvt_ipc_block{s_cap / 2 + src_blocks[i] * half,
                                      d_cap / 2 + dst_blocks[i] * half, half});
        } else {
          // block-major layouts: one contiguous block per tensor
          out.push_back(kvt_ipc_block{src_blocks[i] * B, dst_blocks[i] * B, B});
        }
      }
    }
    if (object_bytes) *object_bytes = obj;
    return KVT_OK;
  });
}

int kvt_enlarge_block_ids(const uint32_t* ids, uint64_t n, uint32_t factor, uint32_t* out) {
  if ((!ids && n) || (!out && n) || factor == 0)
    return fail(KVT_ERR_INVALID, "kvt_enlarge_block_ids: bad argument");
  for (uint64_t i = 0; i < n; ++i) {
    const uint64_t first = static_cast<uint64_t>(ids[i]) * factor;
    if (first + factor - 1 > 0xFFFFFFFFull)
      return fail(KVT_ERR_OVERFLOW, "kvt_enlarge_block_ids: block id does not fit 32 bits");
    for (uint32_t k = 0; k < factor; ++k) out[i * factor + k] = static_cast<uint32_t>(first + k);
  }
  return KVT_OK;
}

}  // extern "C"
