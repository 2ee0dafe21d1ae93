// TEST INFRASTRUCTURE -- not part of the product.
//
// Conversions from the plain-C structs of include/kvt_types.h to the reference's
// C++ types, and the table of the reference's ParseBlock functions by parser id
// (declarations: kvtransfer/include/parse_block_common.h:143-388,
//  kvtransfer/include/parse_block_turboquant.h). Shared by the two checker
// libraries that oracle/Makefile builds from the reference's own sources.
#ifndef KVT_REF_CONVERT_H_
#define KVT_REF_CONVERT_H_

#include <string>
#include <vector>

#include "parse_block_common.h"
#include "parse_block_turboquant.h"

#include "kvt_types.h"

namespace kvt_ref {

using namespace blade_llm;

inline WorkerInfo to_ref(const kvt_worker_info& w) {
  WorkerInfo r;
  r.inst_id = "inst";
  r.worker_id = 0;
  r.engine_tp_size = w.engine_tp_size;
  r.worker_tp_rank = w.worker_tp_rank;
  r.block_sizes.assign(w.block_sizes, w.block_sizes + w.n_tensors);
  r.token_sizes.assign(w.token_sizes, w.token_sizes + w.n_tensors);
  r.layer_num_blocks = w.layer_num_blocks;
  r.num_layers = w.num_layers;
  r.attn_kernel_blk_ntpb = w.attn_kernel_blk_ntpb;
  r.indexer_blk_ntpb = w.indexer_blk_ntpb;
  r.attn_pack_size = w.attn_pack_size;
  r.num_kv_heads = w.num_kv_heads;
  r.num_gdn_layers = w.num_gdn_layers;
  r.hybrid_indexer_token_size = w.hybrid_indexer_token_size;
  r.gdn_conv_elem_size = w.gdn_conv_elem_size;
  r.gdn_ssm_elem_size = w.gdn_ssm_elem_size;
  r.conv_state_shape.assign(w.conv_state_shape, w.conv_state_shape + w.n_conv_state_shape);
  r.ssm_state_shape.assign(w.ssm_state_shape, w.ssm_state_shape + w.n_ssm_state_shape);
  r.gdn_conv_channel_dims.assign(w.gdn_conv_channel_dims,
                                 w.gdn_conv_channel_dims + w.n_gdn_conv_channel_dims);
  r.num_ple_layers = w.num_ple_layers;
  r.ple_block_group = w.ple_block_group;
  r.ple_conv_elem_size = w.ple_conv_elem_size;
  r.ple_conv_state_shape.assign(w.ple_conv_state_shape,
                                w.ple_conv_state_shape + w.n_ple_conv_state_shape);
  r.ple_conv_channel_dims.assign(w.ple_conv_channel_dims,
                                 w.ple_conv_channel_dims + w.n_ple_conv_channel_dims);
  r.kda_conv_dim_first = w.kda_conv_dim_first != 0;
  r.hybrid_attn_token_size = w.hybrid_attn_token_size;
  r.kda_page_stride = w.kda_page_stride;
  return r;
}

inline BlockIds to_groups(const uint32_t* ids, const uint32_t* lens, uint32_t n) {
  BlockIds out(n);
  size_t pos = 0;
  for (uint32_t g = 0; g < n; ++g) {
    out[g].assign(ids + pos, ids + pos + lens[g]);
    pos += lens[g];
  }
  return out;
}

inline ParseBlockFunc pick(int id) {
  switch (id) {
    case KVT_PARSER_RAGGED_PEQD: return parse_block_send_p_eq_d;
    case KVT_PARSER_RAGGED_PGTD: return parse_block_send_p_gt_d;
    case KVT_PARSER_RAGGED_PGTD_DPSK: return parse_block_send_p_gt_d_dpsk;
    case KVT_PARSER_RAGGED_PLTD: return parse_block_send_p_lt_d;
    case KVT_PARSER_FLASH_PEQD: return vllm_parse_block_send_p_eq_d;
    case KVT_PARSER_FLASH_PGTD: return vllm_parse_block_send_p_gt_d;
    case KVT_PARSER_HYBRID_PEQD: return vllm_parse_hybrid_block_send_p_eq_d_block_aligned;
    case KVT_PARSER_HYBRID_PGTD: return vllm_parse_hybrid_block_send_p_gt_d;
    case KVT_PARSER_HYBRID_PLTD: return vllm_parse_hybrid_block_send_p_lt_d;
    case KVT_PARSER_DPSK_PEQD: return vllm_parse_block_send_multi_tensor_p_eq_d;
    case KVT_PARSER_DPSK_PGTD: return vllm_parse_block_send_multi_tensor_p_gt_d;
    case KVT_PARSER_DPSK_PLTD: return vllm_parse_block_send_multi_tensor_p_lt_d;
    case KVT_PARSER_FLASHINFER_PEQD: return vllm_parse_flashinfer_block_send_p_eq_d;
    case KVT_PARSER_FLASHINFER_PGTD: return vllm_parse_flashinfer_block_send_p_gt_d;
    case KVT_PARSER_HYBRID_FI_PEQD: return vllm_parse_qwen3_next_flashinfer_block_send_p_eq_d;
    case KVT_PARSER_HYBRID_FI_PGTD: return vllm_parse_qwen3_next_flashinfer_block_send_p_gt_d;
    case KVT_PARSER_HYBRID_FI_PLTD: return vllm_parse_qwen3_next_flashinfer_block_send_p_lt_d;
    case KVT_PARSER_KDA_PEQD: return parse_kda_block_send_p_eq_d;
    case KVT_PARSER_KDA_PGTD: return parse_kda_block_send_p_gt_d;
    case KVT_PARSER_KDA_PLTD: return parse_kda_block_send_p_lt_d;
    case KVT_PARSER_KIMI_K3_PEQD: return parse_kimi_k3_mla_block_send_p_eq_d;
    case KVT_PARSER_KIMI_K3_PGTD: return parse_kimi_k3_mla_block_send_p_gt_d;
    case KVT_PARSER_KIMI_K3_PLTD: return parse_kimi_k3_mla_block_send_p_lt_d;
    case KVT_PARSER_TURBOQUANT_PEQD: return turboquant_parse_block_send_p_eq_d;
    case KVT_PARSER_TURBOQUANT_PGTD: return turboquant_parse_block_send_p_gt_d;
    default: return nullptr;
  }
}

}  // namespace kvt_ref

#endif  // KVT_REF_CONVERT_H_
