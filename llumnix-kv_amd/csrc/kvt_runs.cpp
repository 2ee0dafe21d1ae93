// Strided run lists: container, expansion to plain ranges, and the inverse
// (finding the arithmetic progressions of a plain list).
#include <cstring>

#include "kvt_internal.h"

namespace kvt {
namespace {

// Same record shape below level `k` (the levels already folded) and nothing
// folded at level k or above yet.
bool same_shape(const kvt_run& a, const kvt_run& b, int k) {
  if (a.length != b.length) return false;
  for (int j = k + 1; j < 3; ++j)
    if (a.n[j] != b.n[j] || a.src_stride[j] != b.src_stride[j] || a.dst_stride[j] != b.dst_stride[j])
      return false;
  return true;
}

// One folding pass: consecutive items of equal shape whose offsets advance by a
// constant, non-negative step on both sides become one item with n[k] = count.
void fold_level(std::vector<kvt_run>& items, int k) {
  size_t w = 0;
  for (size_t i = 0; i < items.size();) {
    kvt_run cur = items[i];
    size_t j = i + 1;
    if (j < items.size() && same_shape(cur, items[j], k) &&
        items[j].src_offset >= cur.src_offset && items[j].dst_offset >= cur.dst_offset) {
      const uint64_t ds = items[j].src_offset - cur.src_offset;
      const uint64_t dd = items[j].dst_offset - cur.dst_offset;
      uint64_t count = 1;
      while (j < items.size() && count < 0xFFFFFFFFull && same_shape(cur, items[j], k) &&
             items[j].src_offset - items[j - 1].src_offset == ds &&
             items[j].dst_offset - items[j - 1].dst_offset == dd &&
             items[j].src_offset >= items[j - 1].src_offset &&
             items[j].dst_offset >= items[j - 1].dst_offset) {
        ++count;
        ++j;
      }
      if (count > 1) {
        cur.n[k] = static_cast<uint32_t>(count);
        cur.src_stride[k] = ds;
        cur.dst_stride[k] = dd;
      }
    }
    items[w++] = cur;
    i = j;
  }
  items.resize(w);
}

// The innermost pass straight from the plain ranges: same rule as fold_level(items, 2),
// without first materialising one 88-byte item per range (a TP-remapping batch has
// hundreds of thousands of ranges, sixteen or more per run).
void fold_ranges(const RunList& v, std::vector<kvt_run>& items) {
  const size_t n = v.size();
  for (size_t i = 0; i < n;) {
    kvt_run cur{};
    cur.src_offset = v[i].src_offset;
    cur.dst_offset = v[i].dst_offset;
    cur.length = v[i].length;
    cur.n[0] = cur.n[1] = cur.n[2] = 1;
    size_t j = i + 1;
    if (j < n && v[j].length == cur.length && v[j].src_offset >= cur.src_offset &&
        v[j].dst_offset >= cur.dst_offset) {
      const uint64_t ds = v[j].src_offset - cur.src_offset;
      const uint64_t dd = v[j].dst_offset - cur.dst_offset;
      uint64_t count = 1;
      while (j < n && count < 0xFFFFFFFFull && v[j].length == cur.length &&
             v[j].src_offset >= v[j - 1].src_offset && v[j].dst_offset >= v[j - 1].dst_offset &&
             v[j].src_offset - v[j - 1].src_offset == ds &&
             v[j].dst_offset - v[j - 1].dst_offset == dd) {
        ++count;
        ++j;
      }
      if (count > 1) {
        cur.n[2] = static_cast<uint32_t>(count);
        cur.src_stride[2] = ds;
        cur.dst_stride[2] = dd;
      }
    }
    items.push_back(cur);
    i = j;
  }
}

}  // namespace
}  // namespace kvt

using namespace kvt;

extern "C" {

int kvt_run_lists_create(kvt_run_lists** out) {
  if (!out) return fail(KVT_ERR_INVALID, "kvt_run_lists_create: null argument");
  *out = new kvt_run_lists();
  return KVT_OK;
}
void kvt_run_lists_destroy(kvt_run_lists* l) { delete l; }
void kvt_run_lists_clear(kvt_run_lists* l) {
  if (l) l->tensors.clear();
}
uint32_t kvt_run_lists_num_tensors(const kvt_run_lists* l) {
  return l ? static_cast<uint32_t>(l->tensors.size()) : 0;
}
int kvt_run_lists_view(const kvt_run_lists* l, uint32_t tensor, const kvt_run** data, uint64_t* n) {
  if (!l || !data || !n) return fail(KVT_ERR_INVALID, "kvt_run_lists_view: null argument");
  if (tensor >= l->tensors.size())
    return fail(KVT_ERR_OUT_OF_RANGE, "kvt_run_lists_view: tensor index out of range");
  *data = l->tensors[tensor].data();
  *n = l->tensors[tensor].size();
  return KVT_OK;
}

int kvt_run_lists_append(kvt_run_lists* l, uint32_t tensor, const kvt_run* runs, uint64_t n) {
  return guarded([&]() -> int {
    if (!l || (!runs && n)) return fail(KVT_ERR_INVALID, "kvt_run_lists_append: null argument");
    if (tensor >= KVT_MAX_TENSORS)
      return fail(KVT_ERR_OUT_OF_RANGE, "kvt_run_lists_append: tensor index out of range");
    for (uint64_t i = 0; i < n; ++i)
      if (runs[i].length == 0 || runs[i].n[0] == 0 || runs[i].n[1] == 0 || runs[i].n[2] == 0)
        return fail(KVT_ERR_INVALID, "kvt_run_lists_append: empty run");
    if (l->tensors.size() <= tensor) l->tensors.resize(tensor + 1);
    l->tensors[tensor].insert(l->tensors[tensor].end(), runs, runs + n);
    return KVT_OK;
  });
}

int kvt_run_lists_totals(const kvt_run_lists* l, uint32_t tensor, uint64_t* n_ranges,
                         uint64_t* n_bytes) {
  if (!l) return fail(KVT_ERR_INVALID, "kvt_run_lists_totals: null argument");
  if (tensor >= l->tensors.size())
    return fail(KVT_ERR_OUT_OF_RANGE, "kvt_run_lists_totals: tensor index out of range");
  uint64_t ranges = 0, bytes = 0;
  for (const kvt_run& r : l->tensors[tensor]) {
    const uint64_t c = static_cast<uint64_t>(r.n[0]) * r.n[1] * r.n[2];
    ranges += c;
    bytes += c * r.length;
  }
  if (n_ranges) *n_ranges = ranges;
  if (n_bytes) *n_bytes = bytes;
  return KVT_OK;
}

int kvt_run_lists_expand(const kvt_run_lists* l, kvt_block_lists* out) {
  return guarded([&]() -> int {
    if (!l || !out) return fail(KVT_ERR_INVALID, "kvt_run_lists_expand: null argument");
    // a run is 88 bytes however many ranges it stands for: refuse to be made to allocate
    // without bound by a few of them
    for (const std::vector<kvt_run>& runs : l->tensors) {
      uint64_t ranges = 0;
      for (const kvt_run& r : runs) {
        uint64_t c = 0;
        if (__builtin_mul_overflow(static_cast<uint64_t>(r.n[0]) * r.n[1], static_cast<uint64_t>(r.n[2]), &c) ||
            __builtin_add_overflow(ranges, c, &ranges) || ranges > (1ull << 31))
          return fail(KVT_ERR_INVALID, "kvt_run_lists_expand: more than 2^31 ranges in one tensor");
      }
    }
    if (out->tensors.size() < l->tensors.size()) out->tensors.resize(l->tensors.size());
    for (size_t t = 0; t < l->tensors.size(); ++t) {
      RunList& dst = out->tensors[t];
      for (const kvt_run& r : l->tensors[t])
        for (uint32_t a = 0; a < r.n[0]; ++a)
          for (uint32_t b = 0; b < r.n[1]; ++b)
            for (uint32_t c = 0; c < r.n[2]; ++c)
              dst.push_back(kvt_ipc_block{
                  r.src_offset + a * r.src_stride[0] + b * r.src_stride[1] + c * r.src_stride[2],
                  r.dst_offset + a * r.dst_stride[0] + b * r.dst_stride[1] + c * r.dst_stride[2],
                  r.length});
    }
    return KVT_OK;
  });
}

int kvt_run_lists_compress(const kvt_block_lists* l, kvt_run_lists* out) {
  return guarded([&]() -> int {
    if (!l || !out) return fail(KVT_ERR_INVALID, "kvt_run_lists_compress: null argument");
    if (out->tensors.size() < l->tensors.size()) out->tensors.resize(l->tensors.size());
    std::vector<kvt_run> items;
    for (size_t t = 0; t < l->tensors.size(); ++t) {
      items.clear();
      fold_ranges(l->tensors[t], items);
      for (int k = 1; k >= 0; --k) fold_level(items, k);
      out->tensors[t].insert(out->tensors[t].end(), items.begin(), items.end());
    }
    return KVT_OK;
  });
}

}  // extern "C"
