// Copy plans: a batch's range lists (or strided runs) cut into chunk tables that
// stay resident on the device, and the pack / unpack launches over them.
#include <algorithm>
#include <cstring>
#include <memory>

#include "kvt_runtime.h"

namespace kvt {
namespace {

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

namespace {
void destroy_slot_plan(kvt_plan* p);
}

// The order of the unpack table and whether every piece is 16-byte aligned throughout.
// What matters most to HBM throughput is that the WRITES of a launch ascend: the unpack table
// is sorted by destination offset (tensor-major: different tensors are different allocations);
// the pack table keeps generation order, which is ascending packed offset (for a merged list
// that is ascending source offset as well). Measured on MI355X: pack of an unmerged batch
// 5.88 -> 6.27 TB/s against sorting the pack table by source offset; unpack +6 % against
// leaving it unsorted.
static int order_pieces(const std::vector<Piece>& pieces, std::vector<uint32_t>& order, bool* all16) {
  static thread_local std::vector<uint64_t> keys;
  const size_t n = pieces.size();
  keys.resize(n);
  for (size_t i = 0; i < n; ++i) {
    if ((pieces[i].src | pieces[i].dst) >> 56)
      return fail(KVT_ERR_INVALID, "kvt_plan_create: offset beyond 2^56");
    keys[i] = (static_cast<uint64_t>(pieces[i].tensor) << 56) | pieces[i].dst;
  }
  stable_order_by_key(keys, order);
  *all16 = true;
  for (size_t i = 0; i < n && *all16; ++i)
    *all16 = ((pieces[i].src | pieces[i].dst | pieces[i].packed | pieces[i].len) & 15u) == 0;
  return KVT_OK;
}

// The two tables: pack order (as generated), unpack order (`order`).
static void build_tables(const std::vector<Piece>& pieces, const std::vector<uint32_t>& order,
                         Chunk* pack_table, Chunk* unpack_table) {
  auto fill = [](Chunk& c, const Piece& q, uint64_t cache) {
    c.cache = cache;
    c.packed = q.packed;
    c.len = q.len;
    c.tensor = q.tensor;
    c.t0 = q.t0;
    c.shape = q.shape;
    c.reserved = 0;
  };
  const size_t n = pieces.size();
  for (size_t i = 0; i < n; ++i) fill(pack_table[i], pieces[i], pieces[i].src);
  for (size_t i = 0; i < n; ++i) fill(unpack_table[i], pieces[order[i]], pieces[order[i]].dst);
}

// Sorts the pieces into the two tables and starts their upload.
static int finish_plan(kvt_plan* p, const std::vector<Piece>& pieces) {
  p->n_chunks = pieces.size();
  if ((p->n_chunks << p->sub_shift) > 0x7FFFFFF0ull)
    return fail(KVT_ERR_INVALID, "kvt_plan_create: too many chunks for one launch");
  static thread_local std::vector<uint32_t> order;
  const size_t n = pieces.size();
  if (int rc = order_pieces(pieces, order, &p->all16)) return rc;
  auto build = [&](Chunk* table) { build_tables(pieces, order, table, table + n); };

  if (p->device == KVT_DEVICE_NONE) {
    p->host_table.resize(2 * n);
    build(p->host_table.data());
    return KVT_OK;
  }
  if (n != 0 && n <= kSmallTable && !p->xform && !p->strided && !p->convert) {
    // short enough to travel in the kernel arguments
    Chunk both[2 * kSmallTable];
    build(both);
    std::memcpy(p->small_pack.c, both, n * sizeof(Chunk));
    std::memcpy(p->small_unpack.c, both + n, n * sizeof(Chunk));
    p->small = true;
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
    // the copy reads the pinned twin and writes the table: the buffer counts as in use by the
    // upload stream until it has run, so destroying the plan early never has to wait for it
    if (e == hipSuccess && p->buf->mark_use(up) != KVT_OK) e = hipErrorUnknown;
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

// The layout transform of a plan: checks it and fills the device-side constants. *half = bytes
// of a K or V half page, *tok_bytes = bytes of one token row over all heads (both 0: none).
static int setup_xform(kvt_plan* p, const kvt_xform* xform, uint64_t* half, uint64_t* tok_bytes) {
  *half = *tok_bytes = 0;
  if (!xform || xform->kind == KVT_XFORM_NONE) return KVT_OK;
  if (xform->kind != KVT_XFORM_HND_NHD) return fail(KVT_ERR_INVALID, "unknown layout transform");
  if (p->n_tensors != 1) return fail(KVT_ERR_INVALID, "layout transform needs a single tensor");
  if (xform->heads == 0 || xform->ntpb == 0 || xform->row_bytes == 0 ||
      xform->row_bytes % 16 != 0 || xform->ntpb > 65535 || xform->heads > 65535)
    return fail(KVT_ERR_INVALID, "layout transform: rows must be multiples of 16 bytes");
  *tok_bytes = static_cast<uint64_t>(xform->heads) * xform->row_bytes;
  *half = *tok_bytes * xform->ntpb;
  p->near = *half < (1ull << 31);
  if (*tok_bytes > kMaxChunk) return fail(KVT_ERR_INVALID, "layout transform: token row too large");
  p->xform = true;
  p->xdev.heads = xform->heads;
  p->xdev.ntpb = xform->ntpb;
  p->xdev.vrow = xform->row_bytes / 16;
  p->xdev.inv_vrow = static_cast<uint32_t>((1ull << 32) / p->xdev.vrow) + 1u;
  p->xdev.inv_heads = static_cast<uint32_t>((1ull << 32) / p->xdev.heads) + 1u;
  return KVT_OK;
}

// Cuts the ranges of `lists` into pieces of at most chunk_bytes for plan p (tensors, capacities
// and transform set) and lays out the packed layer: p->tensor_offset, tensor_bytes, layer_bytes.
static int cut_lists(kvt_plan* p, const kvt_block_lists* lists, uint32_t ntpb, uint64_t half,
                     uint64_t tok_bytes, uint32_t chunk_bytes, std::vector<Piece>& pieces) {
  pieces.clear();
  p->tensor_offset.clear();
  p->tensor_bytes.clear();
  static const RunList kNoRanges;
  uint64_t cursor = 0;
  for (uint32_t t = 0; t < p->n_tensors; ++t) {
    cursor = round_up(cursor, kBlobAlign);
    p->tensor_offset.push_back(cursor);
    uint64_t bad = 0;
    const RunList& runs = t < lists->tensors.size() ? lists->tensors[t] : kNoRanges;
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
          for (uint32_t t0 = 0; t0 < ntpb; t0 += tok_per_chunk) {
            const uint32_t nt = std::min(tok_per_chunk, ntpb - t0);
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
  return KVT_OK;
}

// Plan from plain range lists. object_bytes != 0: the packed side is a sequence of objects of
// object_bytes each, object i placed at i * object_stride (room for the same object of other
// layers behind it); every object must consist of whole ranges.
static int create_plan(int device, const kvt_block_lists* lists, const uint64_t* src_capacity,
                       const uint64_t* dst_capacity, const kvt_xform* xform, uint32_t chunk_bytes,
                       uint64_t object_bytes, uint64_t object_stride, kvt_plan** out) {
  {
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
    if (int rc = setup_xform(p.get(), xform, &half, &tok_bytes)) return rc;

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
    if (int rc = cut_lists(p.get(), lists, p->xform ? xform->ntpb : 0, half, tok_bytes, chunk_bytes, pieces))
      return rc;
    if (object_bytes != 0) {
      // spread the objects: [object 0 of this layer | room for the other layers][object 1 ...
      const uint64_t n_objects = p->tensor_bytes[0] / object_bytes;
      for (Piece& q : pieces) {
        const uint64_t obj = q.packed / object_bytes, in = q.packed % object_bytes;
        if (in + q.len > object_bytes)
          return fail(KVT_ERR_INVALID, "kvt_plan_create_objects: a range straddles two objects");
        q.packed = obj * object_stride + in;
      }
      p->tensor_bytes[0] = n_objects == 0 ? 0 : (n_objects - 1) * object_stride + object_bytes;
      p->layer_bytes = p->tensor_bytes[0];
      p->min_layer_stride = object_bytes;
    } else {
      p->min_layer_stride = p->layer_bytes;
    }
    if (int rc = finish_plan(p.get(), pieces)) return rc;
    *out = p.release();
    return KVT_OK;
  }
}

extern "C" {

// -------------------------------------------------------------------- plan

int kvt_plan_create(int device, const kvt_block_lists* lists, const uint64_t* src_capacity,
                    const uint64_t* dst_capacity, const kvt_xform* xform, uint32_t chunk_bytes,
                    kvt_plan** out) {
  return guarded([&]() -> int {
    return create_plan(device, lists, src_capacity, dst_capacity, xform, chunk_bytes, 0, 0, out);
  });
}

int kvt_plan_create_objects(int device, const kvt_block_lists* lists, const uint64_t* src_capacity,
                            const uint64_t* dst_capacity, uint64_t object_bytes,
                            uint64_t object_stride, uint32_t chunk_bytes, kvt_plan** out) {
  return guarded([&]() -> int {
    if (!lists || lists->tensors.size() != 1)
      return fail(KVT_ERR_INVALID, "kvt_plan_create_objects: exactly one cache tensor per layer");
    if (object_bytes == 0 || object_stride < object_bytes)
      return fail(KVT_ERR_INVALID, "kvt_plan_create_objects: object_stride < object_bytes");
    uint64_t total = 0;
    for (const kvt_ipc_block& r : lists->tensors[0]) total += r.length;
    if (total % object_bytes != 0)
      return fail(KVT_ERR_INVALID, "kvt_plan_create_objects: ranges do not add up to whole objects");
    return create_plan(device, lists, src_capacity, dst_capacity, nullptr, chunk_bytes,
                       object_bytes, object_stride, out);
  });
}

// Cuts the runs of `lists` into pieces for plan p (tensors, capacities and `convert` set): runs
// that stay strided get a record shape (p->shapes) and one piece per chunk of whole outer steps,
// the others are expanded. Lays out the packed layer and sets p->sub_shift for chunk_bytes
// (0: chosen here; fixed_chunk: the caller's size stands, and a record group that does not fit it
// is an error).
static int cut_runs(kvt_plan* p, const kvt_run_lists* lists, uint32_t chunk_bytes, bool fixed_chunk,
                    std::vector<Piece>& pieces) {
  const bool convert = p->convert;
  const uint64_t src_scale = convert ? 2 : 1;  // source bytes per packed byte

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
  p->tensor_offset.clear();
  p->tensor_bytes.clear();
  p->n_strided = 0;
  p->near = true;
  static const std::vector<kvt_run> kNoRuns;
  for (uint32_t t = 0; t < p->n_tensors; ++t) {
    cursor = round_up(cursor, kBlobAlign);
    p->tensor_offset.push_back(cursor);
    uint64_t blob = 0;
    const std::vector<kvt_run>& runs = t < lists->tensors.size() ? lists->tensors[t] : kNoRuns;
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
      uint64_t total = 0, src_len = 0;
      bad = bad || __builtin_mul_overflow(count, r.length, &total) ||
            __builtin_mul_overflow(r.length, src_scale, &src_len) ||
            s_max > p->src_cap[t] || src_len > p->src_cap[t] - s_max ||
            d_max > p->dst_cap[t] || r.length > p->dst_cap[t] - d_max ||
            total > p->dst_cap[t];  // disjoint destination ranges cannot add up to more
      if (bad)
        return fail(KVT_ERR_OUT_OF_RANGE, "kvt_plan_create_runs: run " + std::to_string(ri) +
                                              " of tensor " + std::to_string(t) +
                                              " exceeds the stated capacity");
      if (convert && ((r.src_offset | r.src_stride[0] | r.src_stride[1] | r.src_stride[2]) & 1u))
        return fail(KVT_ERR_INVALID, "kvt_plan_create_runs_bf16_to_fp8: run " + std::to_string(ri) +
                                         " of tensor " + std::to_string(t) +
                                         " does not start on a bf16 element");
      // effective levels (n > 1), outermost first
      int lv[3], n_lv = 0;
      for (int k = 0; k < 3; ++k)
        if (r.n[k] > 1) lv[n_lv++] = k;
      bool strided = n_lv > 0 && r.length < kMinChunk && ((r.length | r.src_offset | r.dst_offset | blob) & 15u) == 0;
      for (int k = 0; k < n_lv && strided; ++k)
        strided = ((r.src_stride[lv[k]] | r.dst_stride[lv[k]]) & 15u) == 0;
      // Kernel nest: the innermost effective level alone when it already spans a slice
      // (folding more levels into the kernel would only multiply record shapes: outer
      // strides between blocks are arbitrary), else the innermost two (K and V of a token
      // inside a token walk). The remaining outer levels are unrolled here.
      const int last = n_lv > 0 ? lv[n_lv - 1] : -1;
      const bool two = n_lv >= 2 && static_cast<uint64_t>(r.n[last]) * r.length < kMinChunk;
      const int in_k = two ? last : -1;
      const int out_k = two ? lv[n_lv - 2] : last;
      const int n_host = n_lv - (two ? 2 : 1);          // levels unrolled on the host: 0..2
      const uint64_t n_in = in_k >= 0 ? r.n[in_k] : 1;
      strided = strided && n_in * r.length <= kMaxChunk / 2;
      uint32_t shape = 0;
      if (strided) {
        StrideShape sh{};
        sh.vlen = static_cast<uint32_t>(r.length >> 4);
        sh.inv_vlen = static_cast<uint32_t>((1ull << 32) / sh.vlen) + 1u;
        sh.n_inner = static_cast<uint32_t>(n_in);
        sh.inv_wlen = static_cast<uint32_t>((1ull << 32) / (4u * sh.vlen)) + 1u;
        sh.inv_inner = sh.n_inner > 1 ? static_cast<uint32_t>((1ull << 32) / sh.n_inner) + 1u : 0u;
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
        const int h0 = n_host >= 1 ? lv[0] : -1, h1 = n_host >= 2 ? lv[1] : -1;
        const uint32_t c0 = h0 >= 0 ? r.n[h0] : 1, c1 = h1 >= 0 ? r.n[h1] : 1;
        for (uint32_t a = 0; a < c0; ++a)
          for (uint32_t b = 0; b < c1; ++b) {
            const uint64_t so = (h0 >= 0 ? a * r.src_stride[h0] : 0) + (h1 >= 0 ? b * r.src_stride[h1] : 0);
            const uint64_t dof = (h0 >= 0 ? a * r.dst_stride[h0] : 0) + (h1 >= 0 ? b * r.dst_stride[h1] : 0);
            spans.push_back(Span{r.src_offset + so, r.dst_offset + dof, blob, sub_bytes, group,
                                 shape, r.src_stride[out_k], r.dst_stride[out_k],
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
  p->min_layer_stride = p->layer_bytes;
  p->strided = n_shapes > 0;

  if (chunk_bytes == 0) {
    std::vector<std::pair<uint64_t, uint64_t>> sized;
    sized.reserve(spans.size());
    for (const Span& sp : spans) sized.emplace_back(sp.bytes, 1);
    chunk_bytes = pick_chunk_bytes(sized);
  }
  if (fixed_chunk && chunk_bytes < max_group)
    return fail(KVT_ERR_INVALID, "a strided record group of " + std::to_string(max_group) +
                                     " bytes does not fit the slot's entries of " +
                                     std::to_string(chunk_bytes) + " bytes");
  while (chunk_bytes < max_group) chunk_bytes *= 2;  // a chunk holds whole outer steps
  p->sub_shift = 0;
  while ((kMinChunk << p->sub_shift) < chunk_bytes) ++p->sub_shift;

  pieces.clear();
  for (const Span& sp : spans) {
    if (sp.group == 0) {
      for (uint64_t o = 0; o < sp.bytes; o += chunk_bytes)
        pieces.push_back(Piece{sp.src + src_scale * o, sp.dst + o, sp.packed + o,
                               static_cast<uint32_t>(std::min<uint64_t>(chunk_bytes, sp.bytes - o)),
                               sp.tensor, 0, 0});
    } else {
      const uint64_t steps_per = chunk_bytes / sp.group;
      const uint64_t per = steps_per * sp.group;
      // how far an entry reaches on the cache side, from its first byte: the pipelined capped
      // kernels address it with 32-bit offsets
      const StrideShape& sh = p->shapes.shape[sp.shape - 1];
      const uint64_t reach = (steps_per - 1) * std::max(sp.s_outer, sp.d_outer) +
                             (sh.n_inner - 1) * std::max(sh.inner[0], sh.inner[1]) +
                             16ull * sh.vlen * src_scale;
      if (reach >= (1ull << 31)) p->near = false;
      for (uint64_t o = 0, step = 0; o < sp.bytes; o += per, step += steps_per) {
        pieces.push_back(Piece{sp.src + step * sp.s_outer, sp.dst + step * sp.d_outer,
                               sp.packed + o,
                               static_cast<uint32_t>(std::min<uint64_t>(per, sp.bytes - o)),
                               sp.tensor, 0, sp.shape});
        ++p->n_strided;
      }
    }
  }
  return KVT_OK;
}

// Plan from strided runs. convert: the pack direction converts bf16 to fp8, every length
// counts fp8 bytes (elements) and the source side reads twice as many bytes.
static int create_runs_plan(int device, const kvt_run_lists* lists, const uint64_t* src_capacity,
                            const uint64_t* dst_capacity, uint32_t chunk_bytes, bool convert,
                            kvt_plan** out) {
  {
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
    p->convert = convert;
    // scratch kept per thread: a plan is built per batch, fresh pages every time would cost
    // more than filling them
    static thread_local std::vector<Piece> pieces;
    if (int rc = cut_runs(p.get(), lists, chunk_bytes, false, pieces)) return rc;
    if (int rc = finish_plan(p.get(), pieces)) return rc;
    *out = p.release();
    return KVT_OK;
  }
}

int kvt_plan_create_runs(int device, const kvt_run_lists* lists, const uint64_t* src_capacity,
                         const uint64_t* dst_capacity, uint32_t chunk_bytes, kvt_plan** out) {
  return guarded([&]() -> int {
    return create_runs_plan(device, lists, src_capacity, dst_capacity, chunk_bytes, false, out);
  });
}

int kvt_plan_create_runs_bf16_to_fp8(int device, const kvt_run_lists* lists,
                                     const uint64_t* src_capacity, const uint64_t* dst_capacity,
                                     uint32_t chunk_bytes, kvt_plan** out) {
  return guarded([&]() -> int {
    return create_runs_plan(device, lists, src_capacity, dst_capacity, chunk_bytes, true, out);
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
  if (p->slot) return destroy_slot_plan(p);
  // No wait for the upload here (on a busy device the copy may sit behind a whole step of
  // kernels that share its hardware queue): the buffer's own record of the upload keeps it
  // out of circulation until the copy has run.
  if (p->uploaded) (void)hipEventDestroy(p->uploaded);
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

}  // extern "C"


// ------------------------------------------------------------------ plan slots

namespace {

void destroy_slot_plan(kvt_plan* p) {
  Slot* sl = p->slot;
  if (sl) {
    for (int i = 0; i < 2; ++i) {
      if (sl->staged[i]) {
        if (sl->staged_rec[i]) (void)hipEventSynchronize(sl->staged[i]);  // the copy reads host[i]
        (void)hipEventDestroy(sl->staged[i]);
      }
      if (sl->host[i]) (void)hipHostFree(sl->host[i]);
    }
    if (sl->filled) (void)hipEventDestroy(sl->filled);
    delete sl;
  }
  if (p->buf) {
    p->buf->wait_idle();
    forget_device_spans();
    p->buf->host = nullptr;  // the staging copies were the slot's
    TablePool::destroy(p->buf);
    delete p->buf;
  }
  delete p;
}

int create_slot(int device, uint32_t n_tensors, const uint64_t* src_capacity, const uint64_t* dst_capacity,
                const kvt_xform* xform, uint32_t chunk_bytes, int kind, uint64_t max_entries,
                uint64_t max_layer_bytes, kvt_plan** out) {
  if (!src_capacity || !dst_capacity || !out)
    return fail(KVT_ERR_INVALID, "kvt_plan_slot_create: null argument");
  if (n_tensors == 0 || n_tensors > KVT_MAX_TENSORS)
    return fail(KVT_ERR_INVALID, "kvt_plan_slot_create: tensor count out of range");
  if (device != KVT_DEVICE_NONE)
    if (int rc = check_device(device)) return rc;
  if (chunk_bytes == 0) chunk_bytes = kMaxAutoChunk;
  const uint32_t max_chunk = kind == kSlotPlain && !(xform && xform->kind != KVT_XFORM_NONE) ? kMaxAutoChunk : kMaxChunk;
  if (chunk_bytes < kMinChunk || chunk_bytes > max_chunk || (chunk_bytes & (chunk_bytes - 1)) != 0)
    return fail(KVT_ERR_INVALID, "kvt_plan_slot_create: chunk_bytes must be a power of two in [4096, " +
                                     std::to_string(max_chunk) + "]");
  if (max_entries == 0 || max_entries > (1ull << 26))
    return fail(KVT_ERR_INVALID, "kvt_plan_slot_create: max_entries must be in [1, 2^26]");

  std::unique_ptr<kvt_plan, void (*)(kvt_plan*)> p(new kvt_plan(), destroy_slot_plan);
  p->device = device;
  p->n_tensors = n_tensors;
  p->src_cap.assign(src_capacity, src_capacity + n_tensors);
  p->dst_cap.assign(dst_capacity, dst_capacity + n_tensors);
  p->tensor_bytes.assign(n_tensors, 0);
  p->tensor_offset.assign(n_tensors, 0);
  p->convert = kind == kSlotConvert;
  p->strided = kind == kSlotStrided || kind == kSlotConvert;
  p->all16 = true;
  p->slot = new Slot();
  Slot* sl = p->slot;
  uint64_t half = 0, tok_bytes = 0;
  if (int rc = setup_xform(p.get(), xform, &half, &tok_bytes)) return rc;
  if (p->xform) {
    if (!p->near) return fail(KVT_ERR_INVALID, "kvt_plan_slot_create: half pages of 2 GiB or more");
    kind = kSlotXform;
    while (chunk_bytes < tok_bytes) chunk_bytes *= 2;  // a chunk holds whole tokens
    sl->ntpb = xform->ntpb;
  }
  sl->kind = kind;
  sl->half = half;
  sl->tok_bytes = tok_bytes;
  sl->chunk_bytes = chunk_bytes;
  while ((kMinChunk << p->sub_shift) < chunk_bytes) ++p->sub_shift;
  if ((max_entries << p->sub_shift) > 0x7FFFFFF0ull)
    return fail(KVT_ERR_INVALID, "kvt_plan_slot_create: too many entries for one launch");
  sl->max_entries = max_entries;
  const uint64_t fits = max_entries * chunk_bytes + kBlobAlign * n_tensors;
  sl->max_layer_bytes = max_layer_bytes ? max_layer_bytes : fits;
  p->min_layer_stride = sl->max_layer_bytes;
  p->layer_bytes = 0;

  if (device == KVT_DEVICE_NONE) {  // for inspection: the tables stay on the host (kvt_plan_host_tables)
    *out = p.release();
    return KVT_OK;
  }
  DeviceGuard g;
  if (int rc = g.enter(device)) return rc;
  // the work counters of the persistent kernels (allocated once per device)
  if (int rc = ticket_pool().prepare(device)) return rc;
  const size_t bytes = kSlotTableOffset + 2 * max_entries * sizeof(Chunk);
  p->buf = new TableBuf();
  p->buf->device = device;
  p->buf->cap = bytes;
  p->buf->captured = true;  // never handed to the pool
  KVT_HIP(hipMalloc(&p->buf->dev, bytes));
  KVT_HIP(hipMemset(p->buf->dev, 0, kSlotTableOffset));  // an empty batch until the first fill
  for (int i = 0; i < 2; ++i) {
    KVT_HIP(hipHostMalloc(reinterpret_cast<void**>(&sl->host[i]), bytes, hipHostMallocDefault));
    std::memset(sl->host[i], 0, kSlotTableOffset);
    KVT_HIP(hipEventCreateWithFlags(&sl->staged[i], hipEventDisableTiming));
  }
  KVT_HIP(hipEventCreateWithFlags(&sl->filled, hipEventDisableTiming));
  p->dev_chunks = reinterpret_cast<Chunk*>(static_cast<uint8_t*>(p->buf->dev) + kSlotTableOffset);
  *out = p.release();
  return KVT_OK;
}

// The second half of a fill: `scratch` holds the batch's layout (cut_lists / cut_runs have
// run on it), `pieces` its table entries. Nothing of the slot has been touched so far.
int fill_slot(kvt_plan* p, kvt_plan& scratch, const std::vector<Piece>& pieces, void* stream,
              kvt_slot_layout* layout) {
  Slot* sl = p->slot;
  const size_t n = pieces.size();
  if (n > sl->max_entries)
    return fail(KVT_ERR_OUT_OF_RANGE, "kvt_plan_slot_fill: the batch needs " + std::to_string(n) +
                                          " table entries, the slot holds " + std::to_string(sl->max_entries));
  if (scratch.layer_bytes > sl->max_layer_bytes)
    return fail(KVT_ERR_OUT_OF_RANGE, "kvt_plan_slot_fill: a packed layer of the batch takes " +
                                          std::to_string(scratch.layer_bytes) + " bytes, the slot was made for " +
                                          std::to_string(sl->max_layer_bytes));
  static thread_local std::vector<uint32_t> order;
  bool all16 = true;
  if (int rc = order_pieces(pieces, order, &all16)) return rc;
  for (uint32_t t = 0; t < p->n_tensors; ++t) all16 = all16 && (scratch.tensor_offset[t] & 15u) == 0;
  if (!all16)
    return fail(KVT_ERR_INVALID, "kvt_plan_slot_fill: a slot moves 16-byte aligned ranges only");
  if (sl->kind != kSlotPlain && sl->kind != kSlotXform && !scratch.near)
    return fail(KVT_ERR_INVALID, "kvt_plan_slot_fill: a table entry spans 2 GiB or more of the cache");
  auto settle = [&]() {  // what the host-side queries answer from now on
    p->n_chunks = n;
    p->tensor_bytes = scratch.tensor_bytes;
    p->tensor_offset = scratch.tensor_offset;
    p->layer_bytes = scratch.layer_bytes;
    p->n_strided = scratch.n_strided;
    if (!layout) return;
    std::memset(layout, 0, sizeof(*layout));
    layout->n_entries = n;
    layout->layer_bytes = scratch.layer_bytes;
    layout->n_tensors = p->n_tensors;
    for (uint32_t t = 0; t < p->n_tensors; ++t) {
      layout->tensor_bytes[t] = scratch.tensor_bytes[t];
      layout->tensor_offset[t] = scratch.tensor_offset[t];
    }
  };
  if (p->device == KVT_DEVICE_NONE) {
    p->host_table.resize(2 * n);
    build_tables(pieces, order, p->host_table.data(), p->host_table.data() + n);
    p->shapes = scratch.shapes;
    settle();
    return KVT_OK;
  }
  DeviceGuard g;
  if (int rc = g.enter(p->device)) return rc;
  const hipStream_t s = static_cast<hipStream_t>(stream);
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &cap) != hipSuccess) (void)hipGetLastError();
  if (cap != hipStreamCaptureStatusNone)
    return fail(KVT_ERR_INVALID, "kvt_plan_slot_fill: not inside a stream capture (fill the slot on the "
                                 "stream that launches the graph, before the launch)");
  std::lock_guard<std::mutex> lock(sl->mu);
  const uint32_t turn = sl->turn;
  if (sl->staged_rec[turn]) KVT_HIP(hipEventSynchronize(sl->staged[turn]));  // two fills ago: its copy has run
  uint8_t* host = sl->host[turn];
  SlotHeader* hdr = reinterpret_cast<SlotHeader*>(host);
  hdr->n_entries = static_cast<uint32_t>(n);
  for (uint32_t t = 0; t < KVT_MAX_TENSORS; ++t)
    hdr->blobs.off[t] = t < p->n_tensors ? scratch.tensor_offset[t] : 0;
  if (p->strided) hdr->shapes = scratch.shapes;
  Chunk* pack_table = reinterpret_cast<Chunk*>(host + kSlotTableOffset);
  Chunk* unpack_table = pack_table + sl->max_entries;
  build_tables(pieces, order, pack_table, unpack_table);
  // eager launches on other streams that still read the old contents come first
  {
    std::lock_guard<std::mutex> uses(p->buf->mu);
    for (const TableBuf::Use& u : p->buf->uses)
      if (u.recorded && u.stream != s) KVT_HIP(hipStreamWaitEvent(s, u.done, 0));
  }
  uint8_t* dev = static_cast<uint8_t*>(p->buf->dev);
  KVT_HIP(hipMemcpyAsync(dev, host, kSlotTableOffset + n * sizeof(Chunk), hipMemcpyHostToDevice, s));
  if (n != 0) {
    const size_t second = kSlotTableOffset + sl->max_entries * sizeof(Chunk);
    KVT_HIP(hipMemcpyAsync(dev + second, host + second, n * sizeof(Chunk), hipMemcpyHostToDevice, s));
  }
  KVT_HIP(hipEventRecord(sl->staged[turn], s));
  sl->staged_rec[turn] = true;
  KVT_HIP(hipEventRecord(sl->filled, s));
  sl->filled_rec = true;
  sl->filled_on = s;
  sl->turn = turn ^ 1u;
  settle();
  return KVT_OK;
}

// The batch-independent part of a slot's plan, copied into the scratch plan a fill cuts into.
void scratch_of(const kvt_plan* p, kvt_plan& scratch) {
  scratch.device = p->device;
  scratch.n_tensors = p->n_tensors;
  scratch.src_cap = p->src_cap;
  scratch.dst_cap = p->dst_cap;
  scratch.xform = p->xform;
  scratch.xdev = p->xdev;
  scratch.convert = p->convert;
  scratch.sub_shift = p->sub_shift;
}

}  // namespace

extern "C" {

int kvt_plan_slot_create(int device, uint32_t n_tensors, const uint64_t* src_capacity,
                         const uint64_t* dst_capacity, const kvt_xform* xform, uint32_t chunk_bytes,
                         uint64_t max_entries, uint64_t max_layer_bytes, kvt_plan** out) {
  return guarded([&]() -> int {
    return create_slot(device, n_tensors, src_capacity, dst_capacity, xform, chunk_bytes, kSlotPlain,
                       max_entries, max_layer_bytes, out);
  });
}

int kvt_plan_slot_create_runs(int device, uint32_t n_tensors, const uint64_t* src_capacity,
                              const uint64_t* dst_capacity, uint32_t chunk_bytes, int bf16_to_fp8,
                              uint64_t max_entries, uint64_t max_layer_bytes, kvt_plan** out) {
  return guarded([&]() -> int {
    return create_slot(device, n_tensors, src_capacity, dst_capacity, nullptr, chunk_bytes,
                       bf16_to_fp8 ? kSlotConvert : kSlotStrided, max_entries, max_layer_bytes, out);
  });
}

int kvt_plan_slot_fill(kvt_plan* p, const kvt_block_lists* lists, void* stream, kvt_slot_layout* layout) {
  return guarded([&]() -> int {
    if (!p || !lists) return fail(KVT_ERR_INVALID, "kvt_plan_slot_fill: null argument");
    if (!p->slot || (p->slot->kind != kSlotPlain && p->slot->kind != kSlotXform))
      return fail(KVT_ERR_INVALID, "kvt_plan_slot_fill: not a plan slot for range lists");
    if (!lists->tensors.empty() && lists->tensors.size() != p->n_tensors)
      return fail(KVT_ERR_INVALID, "kvt_plan_slot_fill: the lists hold " + std::to_string(lists->tensors.size()) +
                                       " tensors, the slot was made for " + std::to_string(p->n_tensors));
    kvt_plan scratch;
    scratch_of(p, scratch);
    static thread_local std::vector<Piece> pieces;
    const Slot* sl = p->slot;
    if (int rc = cut_lists(&scratch, lists, sl->ntpb, sl->half, sl->tok_bytes, sl->chunk_bytes, pieces))
      return rc;
    return fill_slot(p, scratch, pieces, stream, layout);
  });
}

int kvt_plan_slot_fill_runs(kvt_plan* p, const kvt_run_lists* lists, void* stream, kvt_slot_layout* layout) {
  return guarded([&]() -> int {
    if (!p || !lists) return fail(KVT_ERR_INVALID, "kvt_plan_slot_fill_runs: null argument");
    if (!p->slot || (p->slot->kind != kSlotStrided && p->slot->kind != kSlotConvert))
      return fail(KVT_ERR_INVALID, "kvt_plan_slot_fill_runs: not a plan slot for runs");
    if (!lists->tensors.empty() && lists->tensors.size() != p->n_tensors)
      return fail(KVT_ERR_INVALID, "kvt_plan_slot_fill_runs: the lists hold " +
                                       std::to_string(lists->tensors.size()) + " tensors, the slot was made for " +
                                       std::to_string(p->n_tensors));
    kvt_plan scratch;
    scratch_of(p, scratch);
    static thread_local std::vector<Piece> pieces;
    if (int rc = cut_runs(&scratch, lists, p->slot->chunk_bytes, true, pieces)) return rc;
    return fill_slot(p, scratch, pieces, stream, layout);
  });
}

}  // extern "C"

namespace {
// The ticket block of one pipelined launch (nullptr: none to be had, the launch strides).
// An eager launch borrows a block until it has run. A launch that is being recorded into a
// stream capture keeps its block for the life of the plan's table, and shares it with the
// plan's other launches recorded into the same capture on the same stream: those become a
// chain of kernel nodes, which never run at the same time, and each leaves the block zeroed
// (a graph of 80 per-layer launches holds one block, not 80; an engine that captures one graph
// per batch-size bucket would otherwise run the device's 256 capture blocks dry).
struct LaunchTickets {
  int device;
  bool capturing;
  bool shared = false;   // a block this capture already holds: nothing to hand over or back
  uint32_t* block = nullptr;
  LaunchTickets(const kvt_plan* p, int dev, bool cap, hipStream_t s, bool wanted = true)
      : device(dev), capturing(cap) {
    if (!wanted) return;
    if (capturing && p->buf) {
      hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
      unsigned long long id = 0;
      if (hipStreamGetCaptureInfo(s, &st, &id) == hipSuccess && st == hipStreamCaptureStatusActive) {
        std::lock_guard<std::mutex> lock(p->buf->mu);
        for (const TableBuf::CaptureTickets& c : p->buf->capture_tickets)
          if (c.capture == id && c.stream == s) {
            block = c.block;
            shared = true;
            return;
          }
        block = ticket_pool().acquire(dev, true);
        if (block) {
          p->buf->capture_tickets.push_back({id, s, block});
          p->buf->graph_tickets.push_back(block);
          shared = true;   // the table owns it from here on
        }
        return;
      }
      (void)hipGetLastError();
    }
    block = ticket_pool().acquire(dev, cap);
  }
  // the launch is on the stream (or in the graph): eager blocks come back when it has run, a
  // graph's block stays with the plan's table
  void launched(const kvt_plan* p, hipStream_t s) {
    if (!block || shared) return;
    if (!capturing) {
      ticket_pool().launched(device, block, s);
    } else if (p->buf) {
      std::lock_guard<std::mutex> lock(p->buf->mu);
      p->buf->graph_tickets.push_back(block);
    }
    block = nullptr;
  }
  // the launch failed: nothing will ever touch the block
  ~LaunchTickets() {
    if (block && !shared) ticket_pool().give_back(device, block);
  }
};
}  // namespace

// Pack / unpack through a plan slot: always by persistent workgroups over the slot's table, the
// batch's entry count and blob positions read from the header in front of it.
static int run_slot(bool pack, const kvt_plan* p, const kvt_cache* cache, uint32_t first_layer,
                    uint32_t n_layers, void* packed, uint64_t layer_stride, void* stream) {
  Slot* sl = p->slot;
  if (!packed) return fail(KVT_ERR_INVALID, "kvt_pack/unpack: null argument");
  if (p->device != cache->device) return fail(KVT_ERR_INVALID, "plan and cache are on different devices");
  if (p->n_tensors != cache->n_tensors)
    return fail(KVT_ERR_INVALID, "plan and cache disagree on tensors per layer");
  if (static_cast<uint64_t>(first_layer) + n_layers > cache->n_layers)
    return fail(KVT_ERR_OUT_OF_RANGE, "layer range exceeds the registered cache");
  if (n_layers > 65535) return fail(KVT_ERR_INVALID, "at most 65535 layers per launch");
  if (n_layers > 1 && layer_stride < p->min_layer_stride)
    return fail(KVT_ERR_INVALID, "layer_stride smaller than the room the slot was made for");
  const std::vector<uint64_t>& need = pack ? p->src_cap : p->dst_cap;
  for (uint32_t t = 0; t < p->n_tensors; ++t)
    if (cache->capacity[t] < need[t])
      return fail(KVT_ERR_OUT_OF_RANGE, "registered cache is smaller than the plan's capacity");
  if (!cache->aligned16 ||
      ((reinterpret_cast<uintptr_t>(packed) | (n_layers > 1 ? layer_stride : 0)) & 15u) != 0)
    return fail(KVT_ERR_INVALID, "a plan slot needs 16-byte aligned layer tensors, packed buffer and layer stride");
  DeviceGuard g;
  if (int rc = g.enter(p->device)) return rc;
  const hipStream_t s = static_cast<hipStream_t>(stream);
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &cap) != hipSuccess) (void)hipGetLastError();
  const bool capturing = cap != hipStreamCaptureStatusNone;
  bool over_pcie = false;
  if (!capturing && n_layers != 0) {
    uint64_t extent = 0;
    if (__builtin_mul_overflow(static_cast<uint64_t>(n_layers - 1), layer_stride, &extent) ||
        __builtin_add_overflow(extent, sl->max_layer_bytes, &extent))
      return fail(KVT_ERR_OUT_OF_RANGE, "layer stride exceeds 64 bits");
    if (int rc = check_device_span(packed, extent, pack ? "kvt_pack: the packed buffer"
                                                        : "kvt_unpack: the packed buffer", &over_pcie))
      return rc;
    // an eager launch on another stream than the newest fill's waits for that fill
    std::lock_guard<std::mutex> lock(sl->mu);
    if (sl->filled_rec && sl->filled_on != s) KVT_HIP(hipStreamWaitEvent(s, sl->filled, 0));
  }
  const uint32_t cus = device_cu_count(cache->device) & ~7u;
  if (cus < 8) return fail(KVT_ERR_INVALID, "a plan slot needs a device of at least 8 compute units");
  uint32_t max_wgs = copy_wg_cap(cache->device);
  if (over_pcie) max_wgs = max_wgs == 0 ? cus : std::min(max_wgs, cus);  // (see run_plan)
  // Workgroups per CU and tickets: what run_plan gives the same table under a limit (two per CU
  // where a trip moves 8 KiB or an entry goes to one wavefront, else one).
  const bool two_per_cu = p->sub_shift <= 1;
  const uint32_t full = two_per_cu ? 2 * cus : cus;
  const uint32_t wgs = max_wgs == 0 ? full : std::max(8u, std::min(max_wgs & ~7u, full));
  const bool few_pairs = (sl->max_entries << p->sub_shift) * n_layers < (1ull << 31);
  const bool plain = sl->kind == kSlotPlain;
  LaunchTickets tickets(p, cache->device, capturing, s,
                        few_pairs && (plain ? wgs >= full : wgs >= cus && (p->sub_shift >= 2 || wgs >= 2 * cus)));
  const uint8_t* dev = static_cast<const uint8_t*>(p->buf->dev);
  const Chunk* table = p->dev_chunks + (pack ? 0 : sl->max_entries);
  const hipError_t e = launch_slot(sl->kind, pack, table, reinterpret_cast<const SlotHeader*>(dev), p->sub_shift,
                                   cache->dev_ptrs, p->n_tensors, first_layer, n_layers,
                                   static_cast<uint8_t*>(packed), layer_stride, p->xdev, wgs, tickets.block, s);
  if (e != hipSuccess) return hip_fail(e, pack ? "pack launch" : "unpack launch");
  tickets.launched(p, s);
  if (!capturing)
    if (int rc = p->buf->mark_use(s)) return rc;
  return KVT_OK;
}

int kvt::run_plan(bool pack, const kvt_plan* p, const kvt_cache* cache, uint32_t first_layer,
                  uint32_t n_layers, void* packed, uint64_t layer_stride, void* stream,
                  const uint64_t* blob_offsets) {
  if (p && p->slot) {
    if (!cache) return fail(KVT_ERR_INVALID, "kvt_pack/unpack: null argument");
    if (blob_offsets)
      return fail(KVT_ERR_INVALID, "a plan slot's blob positions follow the batch: kvt_pack_at / "
                                   "kvt_unpack_at do not take one");
    return run_slot(pack, p, cache, first_layer, n_layers, packed, layer_stride, stream);
  }
  if (!p || !cache || (!packed && p->n_chunks))
    return fail(KVT_ERR_INVALID, "kvt_pack/unpack: null argument");
  if (p->device == KVT_DEVICE_NONE) return fail(KVT_ERR_INVALID, "a host-only plan cannot be launched");
  if (p->device != cache->device) return fail(KVT_ERR_INVALID, "plan and cache are on different devices");
  if (p->n_tensors != cache->n_tensors)
    return fail(KVT_ERR_INVALID, "plan and cache disagree on tensors per layer");
  if (static_cast<uint64_t>(first_layer) + n_layers > cache->n_layers)
    return fail(KVT_ERR_OUT_OF_RANGE, "layer range exceeds the registered cache");
  if (n_layers > 65535) return fail(KVT_ERR_INVALID, "at most 65535 layers per launch");
  if (n_layers > 1 && !blob_offsets && layer_stride < p->min_layer_stride)
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
  bool over_pcie = false;
  if (!capturing && p->n_chunks != 0 && n_layers != 0) {
    uint64_t extent = 0, layers_span = 0;
    bool wraps = __builtin_mul_overflow(static_cast<uint64_t>(n_layers - 1), layer_stride, &layers_span);
    for (uint32_t t = 0; t < p->n_tensors; ++t) {
      uint64_t end = 0;
      wraps = wraps || __builtin_add_overflow(blobs.off[t], p->tensor_bytes[t], &end);
      extent = std::max(extent, end);
    }
    // a sum that wraps would pass the span check below with a small extent
    if (wraps || __builtin_add_overflow(extent, layers_span, &extent))
      return fail(KVT_ERR_OUT_OF_RANGE, "blob offsets and layer stride exceed 64 bits");
    if (int rc = check_device_span(packed, extent, pack ? "kvt_pack: the packed buffer"
                                                        : "kvt_unpack: the packed buffer", &over_pcie))
      return rc;
  }
  uint32_t max_wgs = copy_wg_cap(cache->device);
  if (over_pcie) {
    // The packed side is pinned host memory: the launch runs at the speed of PCIe, where more
    // than one workgroup per CU only costs (56.4 against 54.9 GB/s on config 2's layers).
    const uint32_t cus = device_cu_count(cache->device) & ~7u;
    if (cus >= 8) max_wgs = max_wgs == 0 ? cus : std::min(max_wgs, cus);
  }
  // A launch whose payload fits the memory-side cache reads with plain loads (kvt_kernels.hip).
  uint64_t payload = 0;
  for (uint32_t t = 0; t < p->n_tensors; ++t) payload += p->tensor_bytes[t];
  // ... and one whose output is read again soon may leave it there (plain stores); not across PCIe
  const uint32_t temporal = (payload * n_layers <= copy_cached_load_max_bytes() ? kPolicyTemporalLoads : 0u) |
                            (!over_pcie && payload * n_layers <= copy_cached_store_max_bytes() ? kPolicyCachedStores : 0u);
  if (p->small) {
    // Under a limit, a 16-byte aligned table goes entry by entry through persistent workgroups
    // like a resident one (below), as soon as there is more than one entry per workgroup
    // (a 64 MiB request, 64 entries x 32 layers, TB/s pack / unpack against the strided loop of
    // the chunk kernel: half the device 4.6 / 4.4 against 4.4 / 4.2, a quarter 4.8 / 4.8 against
    // 4.7 / 4.0, an eighth 4.7 / 4.8 against 4.2 / 3.1, a sixteenth 4.2 / 4.0 against 2.5 / 1.9).
    const uint32_t cus = device_cu_count(cache->device) & ~7u;
    if (max_wgs != 0 && p->all16 && cache->aligned16 && p->sub_shift <= 3 && cus >= 8) {
      uint64_t mis = reinterpret_cast<uintptr_t>(packed) | (n_layers > 1 ? layer_stride : 0);
      for (uint32_t t = 0; t < p->n_tensors; ++t) mis |= blobs.off[t];
      const uint32_t wgs = std::max(8u, std::min(max_wgs & ~7u, p->sub_shift <= 1 ? 2 * cus : cus));
      if ((mis & 15u) == 0 && p->n_chunks * n_layers > wgs) {
        const hipError_t e = launch_copy_entries_small(
            pack, pack ? p->small_pack : p->small_unpack, static_cast<uint32_t>(p->n_chunks),
            p->sub_shift, cache->dev_ptrs, p->n_tensors, first_layer, n_layers,
            static_cast<uint8_t*>(packed), layer_stride, blobs, wgs, s);
        if (e != hipSuccess) return hip_fail(e, pack ? "pack launch" : "unpack launch");
        return KVT_OK;
      }
    }
    // No tickets for a short table: the launch is over before their order pays (a 64 MiB
    // request at half the device: 31 -> 44 us with them); the pipelined loop does pay below
    // half the device (a quarter: 35 -> 30 us, an eighth: 47 -> 34 us).
    const hipError_t e = launch_copy_chunks_small(
        pack, pack ? p->small_pack : p->small_unpack, static_cast<uint32_t>(p->n_chunks),
        p->sub_shift, cache->dev_ptrs, p->n_tensors, first_layer, n_layers,
        static_cast<uint8_t*>(packed), layer_stride, blobs, max_wgs,
        max_wgs < 4u * device_cu_count(cache->device), temporal, nullptr, s);
    if (e != hipSuccess) return hip_fail(e, pack ? "pack launch" : "unpack launch");
    return KVT_OK;
  }
  const Chunk* table = p->dev_chunks + (pack ? 0 : p->n_chunks);
  const uint32_t n = static_cast<uint32_t>(p->n_chunks);
  bool words = false;  // strided chunks moved as 4-byte words instead of 16-byte vectors
  if (p->strided) {
    uint64_t mis = reinterpret_cast<uintptr_t>(packed) | layer_stride | (cache->aligned16 ? 0 : 4);
    for (uint32_t t = 0; t < p->n_tensors; ++t) mis |= blobs.off[t];
    if ((mis & 3u) || !cache->aligned4)
      return fail(KVT_ERR_INVALID,
                  "a strided plan needs 4-byte aligned layer tensors, packed buffer, stride and "
                  "blob offsets (16-byte aligned ones take the fast path)");
    words = (mis & 15u) != 0;
  }
  if (p->convert && pack && p->strided && words)
    return fail(KVT_ERR_INVALID,
                "a converting strided plan needs 16-byte aligned layer tensors, packed buffer, "
                "stride and blob offsets");
  // Tickets count (4 KiB slice, layer) pairs at the finest, in 32 bits.
  const bool few_pairs = (static_cast<uint64_t>(n) << p->sub_shift) * n_layers < (1ull << 31);
  // A capped launch of a plain, fully 16-byte aligned table with entries of 16 or 32 KiB: one
  // persistent workgroup per CU at most (more of them were slower on MI355X: 5.5 TB/s with 256,
  // 5.3 with 512, 5.2 with 1 024), each pipelining whole entries.
  // Entries of 4 or 8 KiB: the same with a wavefront per entry and up to two workgroups per CU
  // (config 4, whose 36 KiB and 8 KiB blocks are cut into 4 KiB entries, TB/s pack / unpack
  // against the strided loop of the chunk kernel: a quarter of the device 6.0 / 5.7 against
  // 5.8 / 5.1, an eighth 5.4 / 5.4 against 4.3 / 3.6, a sixteenth 4.1 / 4.2 against 2.3 / 1.9).
  const bool by_wave = p->sub_shift <= 1;
  // (the unpack of a converting plan moves plain fp8 bytes)
  if (max_wgs != 0 && p->all16 && !(p->convert && pack) && !p->strided && !p->xform &&
      p->sub_shift <= 3 && cache->aligned16 && static_cast<uint64_t>(n) * n_layers > max_wgs) {
    uint64_t mis = reinterpret_cast<uintptr_t>(packed) | (n_layers > 1 ? layer_stride : 0);
    for (uint32_t t = 0; t < p->n_tensors; ++t) mis |= blobs.off[t];
    const uint32_t cus = device_cu_count(cache->device) & ~7u;
    if ((mis & 15u) == 0 && cus >= 8) {
      const uint32_t wgs = std::max(8u, std::min(max_wgs & ~7u, by_wave ? 2 * cus : cus));
      // fewer workgroups than CUs: each has to move more than the ticket's barrier lets it
      // (half the CUs: 4.4 against 5.3 TB/s); a wavefront per entry: the same below two
      // workgroups per CU (one per CU 5.1 / 5.2 with tickets, 5.4 / 5.3 without; two per CU
      // 6.0 / 5.7 with, 5.2 / 5.2 without)
      LaunchTickets tickets(p, cache->device, capturing, s, few_pairs && wgs >= (by_wave ? 2 * cus : cus));
      const hipError_t e = launch_copy_entries(pack, table, n, p->sub_shift, cache->dev_ptrs,
                                               p->n_tensors, first_layer, n_layers,
                                               static_cast<uint8_t*>(packed), layer_stride, blobs,
                                               wgs, tickets.block, s);
      if (e != hipSuccess) return hip_fail(e, pack ? "pack launch" : "unpack launch");
      tickets.launched(p, s);
      if (p->buf) {
        if (capturing) p->buf->captured = true;
        else if (int rc = p->buf->mark_use(s)) return rc;
      }
      return KVT_OK;
    }
  }
  // The same for strided, transposing and converting tables (16-byte vectors only). Measured
  // against the strided loop of the chunk kernels (`for_items`), TB/s pack / unpack on the
  // TP2 -> TP1 batch: half the device 5.9 / 5.9 against 5.8 / 5.9, a quarter 5.9 / 5.9 against
  // 4.4 / 4.2, an eighth 5.9 / 5.8 against 2.5 / 2.4; the converting gather (bytes read and
  // written) 5.9 against 4.3 at one half. Strided entries of 4 or 8 KiB and converting ones of
  // 4096 elements (a sender on TP8: one KV head per rank) go a wavefront per entry, TB/s on a
  // TP8 -> TP1 batch: a quarter 5.6 / 5.3 against 4.0 / 3.6, an eighth 5.5 / 5.1 against
  // 2.5 / 2.2, a sixteenth 3.3 / 3.7 against 1.3 / 1.1; converting gather at a quarter 4.2
  // against 1.9, at an eighth 3.2 against 1.1; transposing half pages of 8 KiB (two KV heads
  // per rank) at a quarter 6.3 / 6.1 against 5.0 / 5.1, at an eighth 5.6 / 5.6 against 3.3 / 3.2.
  const bool converting = p->convert && pack;
  const bool strided_by_wave = p->strided && !converting && !p->xform && p->sub_shift <= 1;
  if (max_wgs != 0 && p->all16 && p->near &&
      (p->strided || p->xform || converting) && !words && p->sub_shift <= 7 && cache->aligned16 && static_cast<uint64_t>(n) * n_layers > max_wgs) {
    uint64_t mis = reinterpret_cast<uintptr_t>(packed) | (n_layers > 1 ? layer_stride : 0);
    for (uint32_t t = 0; t < p->n_tensors; ++t) mis |= blobs.off[t];
    const uint32_t cus = device_cu_count(cache->device) & ~7u;
    if ((mis & 15u) == 0 && cus >= 8) {
      // one workgroup per CU; two where a trip moves only 8 KiB
      const uint32_t per_cu = p->sub_shift <= 1 ? 2u : 1u;
      const uint32_t wgs = std::max(8u, std::min(max_wgs & ~7u, per_cu * cus));
      uint8_t* const pk = static_cast<uint8_t*>(packed);
      // trips of 8 KiB by a single workgroup per CU are better off without the ticket's barrier
      // (converting gather at an eighth of the device: 4.4 against 5.1 TB/s), and so is a grid
      // of fewer workgroups than CUs
      LaunchTickets tickets(p, cache->device, capturing, s,
                            wgs >= cus && few_pairs && (p->sub_shift >= 2 || wgs >= 2 * cus));
      const hipError_t e =
          strided_by_wave ? launch_strided_entries_by_wave(pack, table, n, p->sub_shift, cache->dev_ptrs,
                                              p->n_tensors, first_layer, n_layers, pk, layer_stride, blobs,
                                              p->shapes, wgs, tickets.block, s) :
          converting ? launch_convert_entries(table, n, p->sub_shift, cache->dev_ptrs, p->n_tensors,
                                              first_layer, n_layers, pk, layer_stride, blobs,
                                              p->shapes, wgs, tickets.block, s)
          : p->xform ? launch_xform_entries(pack, table, n, p->sub_shift, cache->dev_ptrs,
                                            p->n_tensors, first_layer, n_layers, pk, layer_stride,
                                            blobs, p->xdev, wgs, tickets.block, s)
                     : launch_strided_entries(pack, table, n, p->sub_shift, cache->dev_ptrs,
                                              p->n_tensors, first_layer, n_layers, pk, layer_stride,
                                              blobs, p->shapes, wgs, tickets.block, s);
      if (e != hipSuccess) return hip_fail(e, pack ? "pack launch" : "unpack launch");
      tickets.launched(p, s);
      if (p->buf) {
        if (capturing) p->buf->captured = true;
        else if (int rc = p->buf->mark_use(s)) return rc;
      }
      return KVT_OK;
    }
  }
  // A launch that ends up capped (more (slice, layer) pairs than the limit) and has at least
  // two workgroups per CU takes its slices by ticket, eight neighbours at a time (config 4,
  // TB/s pack / unpack: half the device 5.6 / 5.5 -> 5.9 / 5.7, a quarter 5.2 / 5.2 ->
  // 5.7 / 5.1; with one workgroup per CU the ticket's barrier costs more than the order
  // brings, 4.4 / 3.4 -> 3.8 / 3.1).
  const uint32_t grid_cap = max_wgs == 0 ? 0u : std::max(8u, max_wgs & ~7u);
  const uint64_t pairs = ((static_cast<uint64_t>(n) << p->sub_shift) + 7u) / 8u * 8u * n_layers;
  const uint32_t n_cus = device_cu_count(cache->device);
  LaunchTickets tickets(p, cache->device, capturing, s,
                        grid_cap != 0 && pairs > grid_cap && few_pairs && n_cus != 0 && grid_cap >= 2 * n_cus);
  uint8_t* const pk8 = static_cast<uint8_t*>(packed);
  const hipError_t e =
      p->convert && pack ? launch_convert_chunks(table, n, p->sub_shift, cache->dev_ptrs,
                                                 p->n_tensors, first_layer, n_layers, pk8,
                                                 layer_stride, blobs, p->shapes, max_wgs,
                                                 tickets.block, s) :
      p->strided ? launch_strided_chunks(pack, table, n, p->sub_shift, cache->dev_ptrs,
                                         p->n_tensors, first_layer, n_layers, pk8, layer_stride,
                                         blobs, p->shapes, words, max_wgs, temporal, tickets.block, s) :
      p->xform ? launch_xform_chunks(pack, table, n, p->sub_shift, cache->dev_ptrs, p->n_tensors,
                                     first_layer, n_layers, pk8, layer_stride, blobs, p->xdev,
                                     max_wgs, temporal, tickets.block, s)
               : launch_copy_chunks(pack, table, n, p->sub_shift, cache->dev_ptrs, p->n_tensors,
                                    first_layer, n_layers, pk8, layer_stride, blobs, max_wgs,
                                    max_wgs < 4u * n_cus, temporal, tickets.block, s);
  if (e == hipSuccess) tickets.launched(p, s);
  if (e != hipSuccess) return hip_fail(e, pack ? "pack launch" : "unpack launch");
  if (p->buf) {
    // remember when the table is last read, so that its storage is not recycled too early
    if (capturing) {
      p->buf->captured = true;
    } else if (int rc = p->buf->mark_use(s)) {
      return rc;
    }
  }
  return KVT_OK;
}

extern "C" {

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
}  // extern "C"
