// TEST INFRASTRUCTURE -- not part of the product.
//
// Drop-in check at the level of the reference's own C++ types: for one case the
// reference's ParseBlockFunc and the replacement handed out by
// llumnix-kv_amd/adapter/kvt_blade_adapter.hpp are called with the very same
// WorkerInfo / ReqSendTask objects and the same send_blocks protocol
// (kvtransfer/src/tx_stub.cpp:201-205); their outputs and the class of the
// exception they throw must be identical. Compiled by oracle/Makefile (target
// `adapter`) with the reference sources where they lie; output in oracle/_ref/.
#include <bitset>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "ref_convert.h"

#include "kvt_blade_adapter.hpp"
#include "kvt_loopback_channel.hpp"

using namespace blade_llm;
using namespace kvt_ref;

namespace {

// 0 ok, 1 out_of_range, 2 overflow_error, 3 other exception
int run(ParseBlockFunc fn, const WorkerInfo& s, const WorkerInfo& d,
        const std::bitset<MAX_TP_SIZE>& valid, uint32_t tp_size, uint32_t tp_rank,
        const std::vector<std::unique_ptr<ReqSendTask>>& tasks,
        std::vector<std::vector<IpcBlock>>& send_blocks) {
  try {
    for (const auto& t : tasks) fn(&s, &d, valid, tp_size, tp_rank, t.get(), send_blocks);
  } catch (const std::out_of_range&) {
    return 1;
  } catch (const std::overflow_error&) {
    return 2;
  } catch (const std::exception&) {
    return 3;
  }
  return 0;
}

}  // namespace

extern "C" {

// Returns 0 when reference and replacement agree; 1 = different exception class,
// 2 = different outer size, 3 = different ranges. *ref_rc = what the reference did
// (0 ok, 1 out_of_range, 2 overflow_error, 3 other), *n_ranges = ranges it produced.
int kvtadp_compare(int parser_id, const kvt_worker_info* src, const kvt_worker_info* dst,
                   uint32_t valid_mask, uint32_t kvt_tp_size, uint32_t kvt_tp_rank,
                   const kvt_task* tasks, uint32_t n_tasks, int* ref_rc, uint64_t* n_ranges) {
  ParseBlockFunc ref_fn = pick(parser_id);
  ParseBlockFunc new_fn = kvt_adapter::parse_block_func(parser_id);
  if (ref_fn == nullptr || new_fn == nullptr) return -1;
  const WorkerInfo s = to_ref(*src), d = to_ref(*dst);
  const std::bitset<MAX_TP_SIZE> valid(valid_mask);
  std::vector<std::unique_ptr<ReqSendTask>> reqs;
  for (uint32_t i = 0; i < n_tasks; ++i) {
    const kvt_task& t = tasks[i];
    auto req = std::make_shared<RequestInfo>(
        "dst", 0u, "req" + std::to_string(i),
        to_groups(t.src_blocks, t.src_group_len, t.n_src_groups),
        to_groups(t.dst_blocks, t.dst_group_len, t.n_dst_groups));
    reqs.emplace_back(new ReqSendTask(req, t.seen_tokens, t.new_tokens, t.reach_last_token != 0));
  }
  std::vector<std::vector<IpcBlock>> a, b;
  const int ra = run(ref_fn, s, d, valid, kvt_tp_size, kvt_tp_rank, reqs, a);
  const int rb = run(new_fn, s, d, valid, kvt_tp_size, kvt_tp_rank, reqs, b);
  *ref_rc = ra;
  uint64_t n = 0;
  for (const auto& v : a) n += v.size();
  *n_ranges = n;
  if (ra != rb) return 1;
  if (ra != 0) return 0;   // what the lists hold after a throw is unspecified
  if (a.size() != b.size()) return 2;
  for (size_t t = 0; t < a.size(); ++t) {
    if (a[t].size() != b[t].size()) return 3;
    for (size_t i = 0; i < a[t].size(); ++i)
      if (a[t][i].src_offset != b[t][i].src_offset || a[t][i].dst_offset != b[t][i].dst_offset ||
          a[t][i].length != b[t][i].length)
        return 3;
  }
  return 0;
}

// Drives kvt_adapter::LoopbackChannel through the IChannel protocol the way
// KvSendStub::TaskContext does (kvtransfer/src/tx_stub.cpp:227-300): connect once, then per
// batch register_data -> send_data(layer) for every layer -> flush. `lists[t]` / `n[t]` are
// tensor t's ranges (written back after register_data, which may merge them in place:
// n[t] receives the new count). kind: 0 PEQD, 1 PLTD, 2 PGTD. alloc / release supply the
// transfer buffer. Returns 0, or 1 out_of_range, 2 overflow_error, 3 other exception;
// metrics (capacity metrics_cap) receives flush()'s string or the exception text.
int kvtadp_loopback_send(int device, void* const* src_layers, const uint64_t* src_capacity,
                         void* const* dst_layers, const uint64_t* dst_capacity,
                         uint32_t n_layers, uint32_t n_tensors, kvt_ipc_block* const* lists,
                         uint64_t* n, int kind, uint32_t batches, void* compute_stream,
                         void* (*alloc)(size_t), void (*release)(void*), char* metrics,
                         size_t metrics_cap) {
  auto say = [&](const std::string& text) {
    if (metrics && metrics_cap) {
      std::strncpy(metrics, text.c_str(), metrics_cap - 1);
      metrics[metrics_cap - 1] = 0;
    }
  };
  try {
    const size_t cells = static_cast<size_t>(n_layers) * n_tensors;
    std::unique_ptr<IChannel> ch(new kvt_adapter::LoopbackChannel(
        device, std::vector<void*>(src_layers, src_layers + cells),
        std::vector<uint64_t>(src_capacity, src_capacity + n_tensors),
        std::vector<void*>(dst_layers, dst_layers + cells),
        std::vector<uint64_t>(dst_capacity, dst_capacity + n_tensors), n_layers, compute_stream,
        alloc, release));
    ch->connect(WorkerInfo("decode-0", 0));
    std::string out;
    for (uint32_t b = 0; b < batches; ++b) {
      std::vector<std::vector<IpcBlock>> data(n_tensors);
      for (uint32_t t = 0; t < n_tensors; ++t)
        for (uint64_t i = 0; i < n[t]; ++i)
          data[t].emplace_back(lists[t][i].src_offset, lists[t][i].dst_offset, lists[t][i].length);
      ch->register_data(data, static_cast<TPKind>(kind));
      for (uint32_t l = 0; l < n_layers; ++l) ch->send_data(l);
      ch->flush(out);
      if (b + 1 == batches)
        for (uint32_t t = 0; t < n_tensors; ++t) {
          n[t] = data[t].size();
          for (size_t i = 0; i < data[t].size(); ++i) {
            lists[t][i].src_offset = data[t][i].src_offset;
            lists[t][i].dst_offset = data[t][i].dst_offset;
            lists[t][i].length = data[t][i].length;
          }
        }
    }
    const bool was_active = ch->is_active();
    ch->close();
    say(out + (was_active && !ch->is_active() ? "closed=1," : "closed=0,"));
    return 0;
  } catch (const std::out_of_range& e) {
    say(e.what());
    return 1;
  } catch (const std::overflow_error& e) {
    say(e.what());
    return 2;
  } catch (const std::exception& e) {
    say(e.what());
    return 3;
  }
}

// The adapter's helper that hands BLLM_KVTRANS_COPY_MEMCPY_* to the library (read from the
// environment at the time of the call). Returns 0, or 1 when it threw.
int kvtadp_apply_copy_memcpy_env(void) {
  try {
    kvt_adapter::apply_copy_memcpy_env();
    return 0;
  } catch (const std::exception&) {
    return 1;
  }
}

}  // extern "C"
