// TEST INFRASTRUCTURE -- not part of the product.
//
// C-ABI shim around the *reference's own* ParseBlock implementation. It is
// compiled (by oracle/Makefile, target `ref`) together with the reference
// sources where they lie under /root/reference/kvtransfer -- nothing of the
// reference is copied into this repository -- and the result goes to
// oracle/_ref/libkvt_ref.so. The shim only converts the plain-C structs of
// include/kvt_types.h into the reference's C++ types and calls the reference
// function selected by `parser_id`
// (declarations: kvtransfer/include/parse_block_common.h:143-388,
//  kvtransfer/include/parse_block_turboquant.h).
//
// Used by tests/ to validate the CPU restatement in oracle/kvt_oracle.cpp and
// by tests/golden/make_golden.py to write golden vectors.
#include <bitset>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "ref_convert.h"
#include "cache_transfer_spec.h"

using namespace blade_llm;
using namespace kvt_ref;

extern "C" {

// Runs the reference parser over `n_tasks` tasks, appending into one
// send_blocks vector exactly as KvSendStub::TaskContext::do_task does
// (kvtransfer/src/tx_stub.cpp:201-205). On success *n_tensors is the outer
// size and out[t] / n_out[t] (t < min(*n_tensors, cap)) is a malloc'd array the
// caller releases with kvtref_free. Returns a KVT_* code.
int kvtref_parse(int parser_id, const kvt_worker_info* src, const kvt_worker_info* dst,
                 uint32_t valid_mask, uint32_t kvt_tp_size, uint32_t kvt_tp_rank,
                 const kvt_task* tasks, uint32_t n_tasks, uint32_t cap,
                 kvt_ipc_block** out, uint64_t* n_out, uint32_t* n_tensors) {
  ParseBlockFunc fn = pick(parser_id);
  if (fn == nullptr) return KVT_ERR_UNSUPPORTED;
  const WorkerInfo s = to_ref(*src);
  const WorkerInfo d = to_ref(*dst);
  const std::bitset<MAX_TP_SIZE> valid(valid_mask);
  std::vector<std::vector<IpcBlock>> send_blocks;
  try {
    for (uint32_t i = 0; i < n_tasks; ++i) {
      const kvt_task& t = tasks[i];
      auto req = std::make_shared<RequestInfo>(
          "dst", 0u, "req" + std::to_string(i),
          to_groups(t.src_blocks, t.src_group_len, t.n_src_groups),
          to_groups(t.dst_blocks, t.dst_group_len, t.n_dst_groups));
      ReqSendTask task(req, t.seen_tokens, t.new_tokens, t.reach_last_token != 0);
      fn(&s, &d, valid, kvt_tp_size, kvt_tp_rank, &task, send_blocks);
    }
  } catch (const std::out_of_range&) {
    return KVT_ERR_OUT_OF_RANGE;
  } catch (const std::overflow_error&) {
    return KVT_ERR_OVERFLOW;
  } catch (const std::exception&) {
    return KVT_ERR_INVALID;
  }
  *n_tensors = static_cast<uint32_t>(send_blocks.size());
  for (uint32_t t = 0; t < send_blocks.size() && t < cap; ++t) {
    const auto& v = send_blocks[t];
    n_out[t] = v.size();
    out[t] = static_cast<kvt_ipc_block*>(std::malloc(sizeof(kvt_ipc_block) * (v.size() + 1)));
    for (size_t i = 0; i < v.size(); ++i) {
      out[t][i].src_offset = v[i].src_offset;
      out[t][i].dst_offset = v[i].dst_offset;
      out[t][i].length = v[i].length;
    }
  }
  return KVT_OK;
}

// The reference's second, descriptor-driven generator (build_transfer_plan +
// generate_all_ipc_blocks, kvtransfer/src/cache_transfer_spec.cpp:293-307, 616-848),
// run over the same tasks. It emits one range per token (and per head), so its
// output equals the hand-written parsers' only after both are normalised; tests
// use it as an independent statement of the byte mapping. *tp_kind receives the
// plan's TPKind.
int kvtref_plan_parse(int cache_shape, const kvt_worker_info* src, const kvt_worker_info* dst,
                      uint32_t valid_mask, uint32_t kvt_tp_size, uint32_t kvt_tp_rank,
                      const kvt_task* tasks, uint32_t n_tasks, uint32_t cap,
                      kvt_ipc_block** out, uint64_t* n_out, uint32_t* n_tensors,
                      int* tp_kind) {
  const WorkerInfo s = to_ref(*src);
  const WorkerInfo d = to_ref(*dst);
  const std::bitset<MAX_TP_SIZE> valid(valid_mask);
  std::vector<std::vector<IpcBlock>> send_blocks;
  try {
    const TransferPlan plan = build_transfer_plan(cache_shape, s, d, valid, kvt_tp_size,
                                                  kvt_tp_rank);
    *tp_kind = static_cast<int>(plan.tpkind);
    for (uint32_t i = 0; i < n_tasks; ++i) {
      const kvt_task& t = tasks[i];
      auto req = std::make_shared<RequestInfo>(
          "dst", 0u, "req" + std::to_string(i),
          to_groups(t.src_blocks, t.src_group_len, t.n_src_groups),
          to_groups(t.dst_blocks, t.dst_group_len, t.n_dst_groups));
      ReqSendTask task(req, t.seen_tokens, t.new_tokens, t.reach_last_token != 0);
      generate_all_ipc_blocks(plan, &task, send_blocks);
    }
  } catch (const std::out_of_range&) {
    return KVT_ERR_OUT_OF_RANGE;
  } catch (const std::overflow_error&) {
    return KVT_ERR_OVERFLOW;
  } catch (const std::exception&) {
    return KVT_ERR_INVALID;
  }
  *n_tensors = static_cast<uint32_t>(send_blocks.size());
  for (uint32_t t = 0; t < send_blocks.size() && t < cap; ++t) {
    const auto& v = send_blocks[t];
    n_out[t] = v.size();
    out[t] = static_cast<kvt_ipc_block*>(std::malloc(sizeof(kvt_ipc_block) * (v.size() + 1)));
    for (size_t i = 0; i < v.size(); ++i) {
      out[t][i].src_offset = v[i].src_offset;
      out[t][i].dst_offset = v[i].dst_offset;
      out[t][i].length = v[i].length;
    }
  }
  return KVT_OK;
}

void kvtref_free(void* p) { std::free(p); }

// The two environment switches the reference latches on first use.
int kvtref_env_bf16_to_fp8(void) { return env_bf162fp8_conversion() ? 1 : 0; }
int kvtref_env_pad_last_attn_block(void) { return env_pad_last_attn_block() ? 1 : 0; }

}  // extern "C"
