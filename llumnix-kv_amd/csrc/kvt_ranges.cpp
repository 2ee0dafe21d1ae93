// Range-list utilities and per-destination dispatch (host side).
#include <algorithm>
#include <limits>
#include <numeric>

#include "kvt_internal.h"

namespace kvt {

namespace {
thread_local std::string g_last_error;
}

int fail(int code, const std::string& msg) {
  g_last_error = msg;
  return code;
}
void clear_error() { g_last_error.clear(); }

void stable_order_by_key(const std::vector<uint64_t>& keys, std::vector<uint32_t>& order) {
  const size_t n = keys.size();
  order.resize(n);
  for (size_t i = 0; i < n; ++i) order[i] = static_cast<uint32_t>(i);
  uint64_t all_or = 0, all_and = ~0ull;
  bool sorted = true;
  for (size_t i = 0; i < n; ++i) {
    all_or |= keys[i];
    all_and &= keys[i];
    if (i && keys[i] < keys[i - 1]) sorted = false;
  }
  if (sorted || n < 2) return;
  const uint64_t varying = all_or ^ all_and;  // bits that differ somewhere
  constexpr int kBits = 11;
  constexpr size_t kBuckets = size_t(1) << kBits;
  // (key, index) pairs move together, so every pass streams through memory; the scratch
  // arrays are kept per thread (a plan is built per batch: no fresh pages every time)
  static thread_local std::vector<uint64_t> ka, kb;
  static thread_local std::vector<uint32_t> ib;
  ka.assign(keys.begin(), keys.end());
  kb.resize(n);
  ib.resize(n);
  uint32_t count[kBuckets];
  for (int shift = 0; shift < 64; shift += kBits) {
    if (((varying >> shift) & (kBuckets - 1)) == 0) continue;
    std::fill(count, count + kBuckets, 0u);
    for (size_t i = 0; i < n; ++i) ++count[(ka[i] >> shift) & (kBuckets - 1)];
    uint32_t run = 0;
    for (size_t k = 0; k < kBuckets; ++k) {
      const uint32_t c = count[k];
      count[k] = run;
      run += c;
    }
    for (size_t i = 0; i < n; ++i) {
      const uint32_t at = count[(ka[i] >> shift) & (kBuckets - 1)]++;
      kb[at] = ka[i];
      ib[at] = order[i];
    }
    ka.swap(kb);
    order.swap(ib);
  }
}

// Sort by source offset (stable) and fold a range into its predecessor when it
// continues it on both sides. Returns {min, max, total, count} of the result.
static void merge_runs(RunList& v, uint64_t stats[4]) {
  if (v.size() > 0xFFFFFFF0ull) throw InvalidError("range list too long");
  {
    static thread_local std::vector<uint64_t> keys;
    static thread_local std::vector<uint32_t> order;
    static thread_local RunList sorted;
    keys.resize(v.size());
    for (size_t i = 0; i < v.size(); ++i) keys[i] = v[i].src_offset;
    stable_order_by_key(keys, order);
    bool identity = true;
    for (size_t i = 0; i < order.size() && identity; ++i) identity = order[i] == i;
    if (!identity) {
      sorted.resize(v.size());
      for (size_t i = 0; i < v.size(); ++i) sorted[i] = v[order[i]];
      v.swap(sorted);   // the caller's old storage becomes next call's scratch
    }
  }
  size_t w = 0;  // index of the run being grown
  for (size_t i = 1; i < v.size(); ++i) {
    kvt_ipc_block& head = v[w];
    const kvt_ipc_block cur = v[i];
    if (cur.src_offset == head.src_offset + head.length &&
        cur.dst_offset == head.dst_offset + head.length) {
      head.length += cur.length;
    } else {
      v[++w] = cur;
    }
  }
  if (!v.empty()) v.resize(w + 1);
  uint64_t mn = std::numeric_limits<uint64_t>::max(), mx = 0, total = 0;
  for (const kvt_ipc_block& b : v) {
    mn = std::min(mn, b.length);
    mx = std::max(mx, b.length);
    total += b.length;
  }
  if (stats) {
    stats[0] = mn;
    stats[1] = mx;
    stats[2] = total;
    stats[3] = v.size();
  }
}

}  // namespace kvt

using namespace kvt;

extern "C" {

const char* kvt_last_error(void) { return g_last_error.c_str(); }

uint64_t kvt_abi_sizeof(int which) {
  switch (which) {
    case 0: return sizeof(kvt_ipc_block);
    case 1: return sizeof(kvt_worker_info);
    case 2: return sizeof(kvt_task);
    case 3: return sizeof(kvt_parse_opts);
    case 4: return sizeof(kvt_xform);
    case 5: return sizeof(kvt_wire_layout);
    case 6: return sizeof(kvt_run);
    default: return 0;
  }
}

uint32_t kvt_compute_valid_ranks_pd(uint32_t p_tp, uint32_t d_tp, int32_t num_kv_heads) {
  p_tp = std::min<uint32_t>(p_tp, KVT_MAX_TP_SIZE);
  const uint32_t everyone = p_tp >= 32 ? 0xFFFFFFFFu : ((1u << p_tp) - 1u);
  // Fan-out (P < D), unknown head count, or at least one distinct head per
  // sender rank: every sender rank carries data nobody else has.
  if (p_tp < d_tp || num_kv_heads <= 0 || static_cast<uint32_t>(num_kv_heads) >= p_tp)
    return everyone;
  const uint32_t heads = static_cast<uint32_t>(num_kv_heads);
  // Heads are replicated over p_tp / heads consecutive ranks. One sender per
  // head when the receiver still splits by head, else one per receiver rank.
  const uint32_t senders = d_tp <= heads ? heads : d_tp;
  const uint32_t stride = p_tp / senders;
  uint32_t mask = 0;
  for (uint32_t i = 0; i < senders; ++i) mask |= 1u << (i * stride);
  return mask;
}

int kvt_select_parser(int cache_shape, const kvt_worker_info* src, const kvt_worker_info* dst,
                      uint32_t* valid_mask, uint32_t* kvt_tp_size, uint32_t* kvt_tp_rank,
                      int* parser_id, int* tp_kind) {
  if (!src || !dst || !valid_mask || !kvt_tp_size || !kvt_tp_rank || !parser_id || !tp_kind)
    return fail(KVT_ERR_INVALID, "kvt_select_parser: null argument");
  if (src->engine_tp_size > KVT_MAX_TP_SIZE || src->worker_tp_rank >= KVT_MAX_TP_SIZE)
    return fail(KVT_ERR_INVALID, "kvt_select_parser: TP size beyond MAX_TP_SIZE");
  const uint32_t valid =
      kvt_compute_valid_ranks_pd(src->engine_tp_size, dst->engine_tp_size, src->num_kv_heads);
  const uint32_t senders = static_cast<uint32_t>(__builtin_popcount(valid));
  *valid_mask = valid;
  *kvt_tp_size = senders;
  *kvt_tp_rank =
      static_cast<uint32_t>(__builtin_popcount(valid & ((1u << src->worker_tp_rank) - 1u)));

  // Shapes that carry TP-sharded linear-attention state pick the TP relation
  // from the engine TP; the others from the number of ranks that really send.
  const bool by_engine_tp = cache_shape == KVT_SHAPE_QWEN3_NEXT_FLASH ||
                            cache_shape == KVT_SHAPE_QWEN3_NEXT_FLASHINFER ||
                            cache_shape == KVT_SHAPE_KIMI_K3_MLA;
  const uint32_t p = by_engine_tp ? src->engine_tp_size : senders;
  const uint32_t d = dst->engine_tp_size;
  enum { EQ = 0, GT = 1, LT = 2 };
  const int rel = p == d ? EQ : (p > d ? GT : LT);

  struct Row {
    int shape;
    int parser[3];  // EQ, GT, LT; -1 = the reference has no parser for it
    int kind[3];
  };
  static const Row table[] = {
      {KVT_SHAPE_RAGGED_FLASH,
       {KVT_PARSER_RAGGED_PEQD, KVT_PARSER_RAGGED_PGTD, KVT_PARSER_RAGGED_PLTD},
       {KVT_TP_PEQD, KVT_TP_PGTD, KVT_TP_PLTD}},
      {KVT_SHAPE_FLASH,
       {KVT_PARSER_FLASH_PEQD, KVT_PARSER_FLASH_PGTD, -1},
       {KVT_TP_PEQD, KVT_TP_PGTD, KVT_TP_UNKNOWN}},
      {KVT_SHAPE_QWEN3_NEXT_FLASH,
       {KVT_PARSER_HYBRID_PEQD, KVT_PARSER_HYBRID_PGTD, KVT_PARSER_HYBRID_PLTD},
       {KVT_TP_PEQD, KVT_TP_PGTD, KVT_TP_PLTD}},
      // sparse MLA is replicated or split per tensor; the transport always
      // treats it as mergeable
      {KVT_SHAPE_DPSK_V32_SPARSE_MLA,
       {KVT_PARSER_DPSK_PEQD, KVT_PARSER_DPSK_PGTD, KVT_PARSER_DPSK_PLTD},
       {KVT_TP_PEQD, KVT_TP_PEQD, KVT_TP_PEQD}},
      {KVT_SHAPE_FLASHINFER,
       {KVT_PARSER_FLASHINFER_PEQD, KVT_PARSER_FLASHINFER_PGTD, -1},
       {KVT_TP_PEQD, KVT_TP_PGTD, KVT_TP_UNKNOWN}},
      {KVT_SHAPE_TURBOQUANT,
       {KVT_PARSER_TURBOQUANT_PEQD, KVT_PARSER_TURBOQUANT_PGTD, -1},
       {KVT_TP_PEQD, KVT_TP_PGTD, KVT_TP_UNKNOWN}},
      {KVT_SHAPE_QWEN3_NEXT_FLASHINFER,
       {KVT_PARSER_HYBRID_FI_PEQD, KVT_PARSER_HYBRID_FI_PGTD, KVT_PARSER_HYBRID_FI_PLTD},
       {KVT_TP_PEQD, KVT_TP_PGTD, KVT_TP_PLTD}},
      {KVT_SHAPE_KIMI_K3_MLA,
       {KVT_PARSER_KIMI_K3_PEQD, KVT_PARSER_KIMI_K3_PGTD, KVT_PARSER_KIMI_K3_PLTD},
       {KVT_TP_PEQD, KVT_TP_PGTD, KVT_TP_PLTD}},
  };
  for (const Row& row : table) {
    if (row.shape != cache_shape) continue;
    int id = row.parser[rel], kind = row.kind[rel];
    if (id < 0) break;
    if (id == KVT_PARSER_RAGGED_PGTD) {
      // replicated (MLA-style) cache: identical rows on both sides, rank 0 sends whole rows
      bool same = src->n_tensors == dst->n_tensors;
      for (uint32_t i = 0; same && i < src->n_tensors; ++i)
        same = src->token_sizes[i] == dst->token_sizes[i];
      if (same) {
        id = KVT_PARSER_RAGGED_PGTD_DPSK;
        kind = KVT_TP_PEQD;
      }
    }
    *parser_id = id;
    *tp_kind = kind;
    return KVT_OK;
  }
  return fail(KVT_ERR_UNSUPPORTED, "unsupported cache_shape");
}

int kvt_merge_interval(kvt_ipc_block* blocks, uint64_t n, uint64_t* n_out, uint64_t stats[4]) {
  return guarded([&]() -> int {
    if ((!blocks && n) || !n_out) return fail(KVT_ERR_INVALID, "kvt_merge_interval: null argument");
    RunList v(blocks, blocks + n);
    merge_runs(v, stats);
    std::copy(v.begin(), v.end(), blocks);
    *n_out = v.size();
    return KVT_OK;
  });
}

int kvt_block_lists_merge(kvt_block_lists* l) {
  return guarded([&]() -> int {
    if (!l) return fail(KVT_ERR_INVALID, "kvt_block_lists_merge: null argument");
    for (RunList& v : l->tensors) merge_runs(v, nullptr);
    return KVT_OK;
  });
}

int kvt_validate_ipc_block_bounds(const kvt_ipc_block* blocks, uint64_t n, uint64_t capacity,
                                  int which, uint64_t length_scale, uint64_t* bad_idx) {
  if (!blocks && n) return fail(KVT_ERR_INVALID, "kvt_validate_ipc_block_bounds: null argument");
  for (uint64_t i = 0; i < n; ++i) {
    const uint64_t off = which == 0 ? blocks[i].src_offset : blocks[i].dst_offset;
    const uint64_t len = blocks[i].length;
    bool ok = len != 0 && length_scale != 0 && off <= capacity;
    if (ok) {
      const uint64_t room = capacity - off;  // no overflow: off <= capacity
      ok = len <= room / length_scale;       // <=> len * scale <= room, overflow-free
    }
    if (!ok) {
      if (bad_idx) *bad_idx = i;
      return fail(KVT_ERR_OUT_OF_RANGE, "KVT GPU buffer range validation failed");
    }
  }
  return KVT_OK;
}

}  // extern "C"
