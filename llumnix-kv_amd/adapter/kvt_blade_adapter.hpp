// Source-level glue between Blade-KVT's own C++ types and libkvt_hip's C ABI.
//
// This header is compiled INSIDE the Blade-KVT tree (it includes the reference's
// common.h / channel.h / parse_block_common.h / envcfg.h, which are not part of
// this repository) and gives a maintainer ready-made replacements with the
// reference's exact signatures:
//
//   kvt_adapter::parse_block_func(id)   -> a ParseBlockFunc
//                                          (kvtransfer/include/parse_block_common.h:86-94)
//   kvt_adapter::select(...)            -> what the if/else ladder of
//                                          TaskContext::refresh_dst_info computes
//                                          (kvtransfer/src/tx_stub.cpp:417-591)
//   kvt_adapter::merge_interval(v)      -> merge_interval + erase of empty entries
//                                          (kvtransfer/src/channel.cpp:53-98)
//   kvt_adapter::validate_ipc_block_bounds(...)
//                                          (kvtransfer/src/channel.cpp:11-51)
//
// Errors cross the boundary as the exception classes the reference throws
// (std::out_of_range, std::overflow_error, std::runtime_error), so do_task()'s
// catch block (kvtransfer/src/tx_stub.cpp:214-225) keeps working unchanged.
#ifndef KVT_BLADE_ADAPTER_HPP_
#define KVT_BLADE_ADAPTER_HPP_

#include <bitset>
#include <cstdlib>
#include <cstring>
#include <stdexcept>
#include <string>
#include <tuple>
#include <utility>
#include <vector>

#include "channel.h"
#include "common.h"
#include "envcfg.h"
#include "parse_block_common.h"

#include "kvt_hip.h"

namespace kvt_adapter {

static_assert(sizeof(blade_llm::IpcBlock) == sizeof(kvt_ipc_block), "IpcBlock layout differs");

inline void raise(int rc) {
  const std::string msg = kvt_last_error();
  switch (rc) {
    case KVT_OK: return;
    case KVT_ERR_OUT_OF_RANGE: throw std::out_of_range(msg);
    case KVT_ERR_OVERFLOW: throw std::overflow_error(msg);
    default: throw std::runtime_error(msg);
  }
}

template <class V, class T>
inline void copy_dims(const V& from, T* to, uint32_t* count, size_t cap, const char* what) {
  if (from.size() > cap) throw std::runtime_error(std::string("kvt adapter: too many entries in ") + what);
  *count = static_cast<uint32_t>(from.size());
  for (size_t i = 0; i < from.size(); ++i) to[i] = static_cast<T>(from[i]);
}

inline kvt_worker_info to_kvt(const blade_llm::WorkerInfo& w) {
  kvt_worker_info k;
  std::memset(&k, 0, sizeof(k));
  k.engine_tp_size = w.engine_tp_size;
  k.worker_tp_rank = w.worker_tp_rank;
  uint32_t n_tok = 0;
  copy_dims(w.block_sizes, k.block_sizes, &k.n_tensors, KVT_MAX_TENSORS, "block_sizes");
  copy_dims(w.token_sizes, k.token_sizes, &n_tok, KVT_MAX_TENSORS, "token_sizes");
  k.layer_num_blocks = static_cast<uint32_t>(w.layer_num_blocks);
  k.num_layers = static_cast<uint32_t>(w.num_layers);
  k.attn_kernel_blk_ntpb = w.attn_kernel_blk_ntpb;
  k.indexer_blk_ntpb = w.indexer_blk_ntpb;
  k.attn_pack_size = w.attn_pack_size;
  k.num_kv_heads = w.num_kv_heads;
  k.num_gdn_layers = w.num_gdn_layers;
  k.hybrid_indexer_token_size = w.hybrid_indexer_token_size;
  k.gdn_conv_elem_size = w.gdn_conv_elem_size;
  k.gdn_ssm_elem_size = w.gdn_ssm_elem_size;
  copy_dims(w.conv_state_shape, k.conv_state_shape, &k.n_conv_state_shape, KVT_MAX_SHAPE_DIMS,
            "conv_state_shape");
  copy_dims(w.ssm_state_shape, k.ssm_state_shape, &k.n_ssm_state_shape, KVT_MAX_SHAPE_DIMS,
            "ssm_state_shape");
  copy_dims(w.gdn_conv_channel_dims, k.gdn_conv_channel_dims, &k.n_gdn_conv_channel_dims,
            KVT_MAX_CHANNEL_DIMS, "gdn_conv_channel_dims");
  k.num_ple_layers = w.num_ple_layers;
  k.ple_block_group = w.ple_block_group;
  k.ple_conv_elem_size = w.ple_conv_elem_size;
  copy_dims(w.ple_conv_state_shape, k.ple_conv_state_shape, &k.n_ple_conv_state_shape,
            KVT_MAX_SHAPE_DIMS, "ple_conv_state_shape");
  copy_dims(w.ple_conv_channel_dims, k.ple_conv_channel_dims, &k.n_ple_conv_channel_dims,
            KVT_MAX_CHANNEL_DIMS, "ple_conv_channel_dims");
  k.kda_conv_dim_first = w.kda_conv_dim_first ? 1u : 0u;
  k.hybrid_attn_token_size = w.hybrid_attn_token_size;
  k.kda_page_stride = w.kda_page_stride;
  return k;
}

// One compiled parser per calling thread, rebuilt when the destination changes
// (do_task() calls the function once per request with identical arguments).
struct ParserSlot {
  int id = -1;
  kvt_worker_info src, dst;
  uint32_t valid = 0, tp_size = 0, tp_rank = 0;
  kvt_parse_opts opts{0, 1};
  kvt_parser* parser = nullptr;
  kvt_block_lists* lists = nullptr;
  std::vector<uint32_t> ids[2], lens[2];
  ~ParserSlot() {
    kvt_parser_destroy(parser);
    kvt_block_lists_destroy(lists);
  }
};

inline void flatten(const blade_llm::BlockIds& groups, std::vector<uint32_t>& ids,
                    std::vector<uint32_t>& lens) {
  ids.clear();
  lens.clear();
  for (const auto& g : groups) {
    lens.push_back(static_cast<uint32_t>(g.size()));
    ids.insert(ids.end(), g.begin(), g.end());
  }
}

template <int ID>
void parse_block(const blade_llm::WorkerInfo* src, const blade_llm::WorkerInfo* dst,
                 const std::bitset<blade_llm::MAX_TP_SIZE>& valid_ranks, uint32_t kvt_tp_size,
                 uint32_t kvt_tp_rank, const blade_llm::ReqSendTask* task,
                 std::vector<std::vector<blade_llm::IpcBlock>>& send_blocks) {
  static thread_local ParserSlot slot;
  const kvt_worker_info ks = to_kvt(*src), kd = to_kvt(*dst);
  const uint32_t valid = static_cast<uint32_t>(valid_ranks.to_ulong());
  const kvt_parse_opts opts{blade_llm::env_bf162fp8_conversion() ? 1u : 0u,
                            blade_llm::env_pad_last_attn_block() ? 1u : 0u};
  if (slot.parser == nullptr || slot.id != ID || std::memcmp(&slot.src, &ks, sizeof(ks)) != 0 ||
      std::memcmp(&slot.dst, &kd, sizeof(kd)) != 0 || slot.valid != valid ||
      slot.tp_size != kvt_tp_size || slot.tp_rank != kvt_tp_rank ||
      std::memcmp(&slot.opts, &opts, sizeof(opts)) != 0) {
    kvt_parser_destroy(slot.parser);
    slot.parser = nullptr;
    raise(kvt_parser_create(ID, &ks, &kd, valid, kvt_tp_size, kvt_tp_rank, &opts, &slot.parser));
    slot.id = ID;
    slot.src = ks;
    slot.dst = kd;
    slot.valid = valid;
    slot.tp_size = kvt_tp_size;
    slot.tp_rank = kvt_tp_rank;
    slot.opts = opts;
  }
  if (slot.lists == nullptr) raise(kvt_block_lists_create(&slot.lists));
  kvt_block_lists_clear(slot.lists);
  flatten(task->src_blocks(), slot.ids[0], slot.lens[0]);
  flatten(task->dst_blocks(), slot.ids[1], slot.lens[1]);
  kvt_task t;
  std::memset(&t, 0, sizeof(t));
  t.seen_tokens = task->seen_tokens;
  t.new_tokens = task->new_tokens;
  t.reach_last_token = task->reach_last_token ? 1u : 0u;
  t.n_src_groups = static_cast<uint32_t>(slot.lens[0].size());
  t.n_dst_groups = static_cast<uint32_t>(slot.lens[1].size());
  t.src_blocks = slot.ids[0].data();
  t.src_group_len = slot.lens[0].data();
  t.dst_blocks = slot.ids[1].data();
  t.dst_group_len = slot.lens[1].data();
  const int rc = kvt_parse_block(slot.parser, &t, slot.lists);
  // append what was produced (also the part before a failing range, as the reference does)
  const uint32_t n = kvt_block_lists_num_tensors(slot.lists);
  if (n != 0 && send_blocks.size() != n) send_blocks.resize(n);
  for (uint32_t i = 0; i < n; ++i) {
    const kvt_ipc_block* data = nullptr;
    uint64_t count = 0;
    raise(kvt_block_lists_view(slot.lists, i, &data, &count));
    auto& out = send_blocks[i];
    out.reserve(out.size() + count);
    for (uint64_t j = 0; j < count; ++j)
      out.emplace_back(data[j].src_offset, data[j].dst_offset, data[j].length);
  }
  raise(rc);
}

namespace detail {
template <int... I>
inline blade_llm::ParseBlockFunc table_lookup(int id, std::integer_sequence<int, I...>) {
  static const blade_llm::ParseBlockFunc table[] = {&parse_block<I>...};
  return (id >= 0 && id < static_cast<int>(sizeof...(I))) ? table[id] : nullptr;
}
}  // namespace detail

// The replacement for one of the reference's ParseBlockFunc implementations
// (ids: KVT_PARSER_*, one per reference function).
inline blade_llm::ParseBlockFunc parse_block_func(int parser_id) {
  return detail::table_lookup(parser_id, std::make_integer_sequence<int, KVT_PARSER_COUNT>());
}

struct Selection {
  std::bitset<blade_llm::MAX_TP_SIZE> valid_ranks;
  uint32_t kvt_tp_size = 0, kvt_tp_rank = 0;
  blade_llm::ParseBlockFunc parse_block = nullptr;
  blade_llm::TPKind tp_kind = blade_llm::TPKind::UNKNOWN;
};

// refresh_dst_info()'s selection for a destination. Throws std::runtime_error
// ("unsupported cache_shape") like the reference.
inline Selection select(int cache_shape, const blade_llm::WorkerInfo& src,
                        const blade_llm::WorkerInfo& dst) {
  const kvt_worker_info ks = to_kvt(src), kd = to_kvt(dst);
  uint32_t valid = 0;
  int parser_id = -1, kind = KVT_TP_UNKNOWN;
  Selection s;
  raise(kvt_select_parser(cache_shape, &ks, &kd, &valid, &s.kvt_tp_size, &s.kvt_tp_rank,
                          &parser_id, &kind));
  s.valid_ranks = std::bitset<blade_llm::MAX_TP_SIZE>(valid);
  s.parse_block = parse_block_func(parser_id);
  s.tp_kind = static_cast<blade_llm::TPKind>(kind);   // same numbering (channel.h:51-56)
  return s;
}

// merge_interval plus the removal of emptied entries that its callers perform
// (kvtransfer/src/tcp_channel.cpp:376-392). Returns {min, max, total, count}.
inline std::tuple<size_t, size_t, size_t, size_t> merge_interval(
    std::vector<blade_llm::IpcBlock>& input) {
  uint64_t n_out = 0, stats[4] = {0, 0, 0, 0};
  raise(kvt_merge_interval(reinterpret_cast<kvt_ipc_block*>(input.data()), input.size(), &n_out,
                           stats));
  input.erase(input.begin() + static_cast<std::ptrdiff_t>(n_out), input.end());
  return {stats[0], stats[1], stats[2], stats[3]};
}

inline void validate_ipc_block_bounds(const std::vector<blade_llm::IpcBlock>& blocks,
                                      size_t capacity, blade_llm::IpcBlockOffset kind,
                                      size_t length_scale = 1) {
  uint64_t bad = 0;
  raise(kvt_validate_ipc_block_bounds(reinterpret_cast<const kvt_ipc_block*>(blocks.data()),
                                      blocks.size(), capacity,
                                      kind == blade_llm::IpcBlockOffset::DESTINATION ? 1 : 0,
                                      length_scale, &bad));
}

// get_kernel_copy_buffer (kvtransfer/include/copy_utils.h:127): the calling thread's
// {device, pinned host} metadata buffers; {nullptr, nullptr} on failure like the reference.
inline std::pair<char*, char*> get_kernel_copy_buffer(int device_id, int64_t max_block_num = 0) {
  int64_t *dev = nullptr, *host = nullptr;
  if (kvt_get_kernel_copy_buffer(device_id, max_block_num, &dev, &host) != KVT_OK)
    return {nullptr, nullptr};
  return {reinterpret_cast<char*>(dev), reinterpret_cast<char*>(host)};
}

// get_thread_local_h2d_stream / _d2h_stream (copy_utils.h:128-129) as void* stream handles.
inline void* get_thread_local_h2d_stream(int device_id) {
  void* s = nullptr;
  raise(kvt_get_thread_local_stream(device_id, KVT_COPY_H2D, &s));
  return s;
}
inline void* get_thread_local_d2h_stream(int device_id) {
  void* s = nullptr;
  raise(kvt_get_thread_local_stream(device_id, KVT_COPY_D2H, &s));
  return s;
}

// What CopyKernelConfig::initialize does with BLLM_KVTRANS_KERNEL_COPY_SM_USAGE
// (kvtransfer/src/copy_kernels.cpp:327-335): hand the configured share to the library, once,
// where the reference initialises its copy threads.
inline void apply_kernel_copy_sm_usage(int device_id) {
  raise(kvt_set_copy_cu_usage(device_id, blade_llm::env_kernel_copy_sm_usage()));
}

// BLLM_KVTRANS_COPY_MEMCPY_BLOCK_THRESHOLD_BYTES / BLLM_KVTRANS_COPY_MEMCPY_MAX_BLOCKS
// (kvtransfer/src/copy_kernels.cpp:496-499), when set, replace the library's own thresholds
// for handing a list to the DMA engines; unset or unparsable values leave them alone (and
// with neither set the library's start-up measurement stays free to choose them).
inline void apply_copy_memcpy_env() {
  uint64_t min_bytes = 0, max_ranges = 0;
  raise(kvt_get_copy_memcpy_thresholds(&min_bytes, &max_ranges));
  auto read = [](const char* name, uint64_t* out) {
    const char* v = std::getenv(name);
    if (v == nullptr || *v == '\0') return false;
    char* end = nullptr;
    const unsigned long long x = std::strtoull(v, &end, 10);
    if (end == v || *end != '\0') return false;
    *out = x;
    return true;
  };
  const bool a = read("BLLM_KVTRANS_COPY_MEMCPY_BLOCK_THRESHOLD_BYTES", &min_bytes);
  const bool b = read("BLLM_KVTRANS_COPY_MEMCPY_MAX_BLOCKS", &max_ranges);
  if (!a && !b) return;
  if (min_bytes == 0) min_bytes = 1;
  raise(kvt_set_copy_memcpy_thresholds(min_bytes, max_ranges));
}

// initialize_copy_method_profile as the reference's copy threads call it
// (kvtransfer/src/copy_utils.cpp:52): BLLM_KVTRANS_COPY_PROFILE_ENABLE=0 skips the
// measurement (kvtransfer/src/copy_kernels.cpp:501-508) and leaves the thresholds as they are.
inline void initialize_copy_method_profile(int device_id) {
  const char* v = std::getenv("BLLM_KVTRANS_COPY_PROFILE_ENABLE");
  if (v != nullptr && std::atoi(v) == 0) return;  // env_bool, copy_kernels.cpp:168-174
  raise(kvt_initialize_copy_method_profile(device_id));
}

}  // namespace kvt_adapter

#endif  // KVT_BLADE_ADAPTER_HPP_
