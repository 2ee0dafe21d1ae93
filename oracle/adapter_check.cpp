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
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "ref_convert.h"

#include "kvt_blade_adapter.hpp"

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

}  // extern "C"
