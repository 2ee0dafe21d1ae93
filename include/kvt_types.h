/*
 * kvt_types.h -- plain-C data types shared by every entry point of the
 * MI355X KV-cache pack/unpack library.
 *
 * All structs are PODs with fixed-size inline arrays (no pointers except in
 * kvt_task) so that they can cross a C ABI and be filled from ctypes / cgo /
 * JNI without marshalling helpers.
 *
 * Reference types these mirror (paths relative to the reference checkout):
 *   kvt_ipc_block    <- struct IpcBlock           kvtransfer/include/channel.h:15-21
 *   kvt_worker_info  <- struct WorkerInfo         kvtransfer/include/common.h:117-211
 *   kvt_task         <- class ReqSendTask +       kvtransfer/include/common.h:224-262
 *                       RequestInfo::src_blocks / dst_blocks (:275-276)
 *   KVT_SHAPE_*      <- cache-shape constants     kvtransfer/include/envcfg.h:25-52
 *   KVT_TP_*         <- enum class TPKind         kvtransfer/include/channel.h:51-56
 *   KVT_MAX_TP_SIZE  <- MAX_TP_SIZE               kvtransfer/include/envcfg.h:79
 */
#ifndef KVT_TYPES_H_
#define KVT_TYPES_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KVT_MAX_TP_SIZE 16
#define KVT_MAX_TENSORS 8   /* cache tensors per layer (1 for most shapes, 2 for sparse MLA) */
#define KVT_MAX_SHAPE_DIMS 4
#define KVT_MAX_CHANNEL_DIMS 8

/* One byte-range copy: src_offset/dst_offset are relative to the layer tensor
 * base on the sending / receiving side; the same list is replayed per layer. */
typedef struct kvt_ipc_block {
  uint64_t src_offset;
  uint64_t dst_offset;
  uint64_t length;
} kvt_ipc_block;

/* A strided nest of equal-length ranges: n[0]*n[1]*n[2] ranges of `length`
 * bytes; the range with indices (i0, i1, i2), i2 running fastest, is
 *   (src_offset + sum_k i_k*src_stride[k], dst_offset + sum_k i_k*dst_stride[k], length).
 * Expanding the runs of a list in order gives exactly the kvt_ipc_block list
 * (same order, hence the same packed blob). A TP-remapping parser emits one run
 * per block segment instead of one range per token (and per head). No reference
 * counterpart: the reference materialises every range on the host
 * (e.g. parse_block_send_gt, kvtransfer/src/parse_block_common.cpp:81-129). */
typedef struct kvt_run {
  uint64_t src_offset;
  uint64_t dst_offset;
  uint64_t length;
  uint32_t n[3];
  uint32_t reserved0;
  uint64_t src_stride[3];
  uint64_t dst_stride[3];
} kvt_run;

/* Cache shapes (values equal the reference's BLLM_KVTRANS_CACHE_SHAPE ids). */
enum {
  KVT_SHAPE_RAGGED_FLASH = 1,          /* [nblk, bs, 2, h, d] ; also dense MLA [nblk, bs, d] */
  KVT_SHAPE_FLASH = 2,                 /* [2, nblk, bs, h, d]                                */
  KVT_SHAPE_QWEN3_NEXT_FLASH = 3,      /* hybrid pages: GDN state pages + NHD attn pages     */
  KVT_SHAPE_DPSK_V32_SPARSE_MLA = 4,   /* two 3-D tensors per layer (MLA latent + indexer)   */
  KVT_SHAPE_FLASHINFER = 5,            /* [nblk, 2, h, bs, d] (HND)                          */
  KVT_SHAPE_TURBOQUANT = 6,            /* alias of the hybrid page parsers                   */
  KVT_SHAPE_QWEN3_NEXT_FLASHINFER = 7, /* hybrid pages with HND attn pages                   */
  KVT_SHAPE_KIMI_K3_MLA = 8            /* KDA state groups + replicated MLA prefix           */
};

/* Relation between the sender's effective TP and the receiver's TP. */
enum {
  KVT_TP_PEQD = 0,
  KVT_TP_PLTD = 1,
  KVT_TP_PGTD = 2,
  KVT_TP_UNKNOWN = 3
};

/* Parser ids: one per reference ParseBlockFunc implementation
 * (kvtransfer/include/parse_block_common.h:143-388,
 *  kvtransfer/include/parse_block_turboquant.h). */
enum {
  KVT_PARSER_RAGGED_PEQD = 0,       /* parse_block_send_p_eq_d                              */
  KVT_PARSER_RAGGED_PGTD = 1,       /* parse_block_send_p_gt_d                              */
  KVT_PARSER_RAGGED_PGTD_DPSK = 2,  /* parse_block_send_p_gt_d_dpsk                         */
  KVT_PARSER_RAGGED_PLTD = 3,       /* parse_block_send_p_lt_d                              */
  KVT_PARSER_FLASH_PEQD = 4,        /* vllm_parse_block_send_p_eq_d                         */
  KVT_PARSER_FLASH_PGTD = 5,        /* vllm_parse_block_send_p_gt_d                         */
  KVT_PARSER_HYBRID_PEQD = 6,       /* vllm_parse_hybrid_block_send_p_eq_d_block_aligned    */
  KVT_PARSER_HYBRID_PGTD = 7,       /* vllm_parse_hybrid_block_send_p_gt_d                  */
  KVT_PARSER_HYBRID_PLTD = 8,       /* vllm_parse_hybrid_block_send_p_lt_d                  */
  KVT_PARSER_DPSK_PEQD = 9,         /* vllm_parse_block_send_multi_tensor_p_eq_d            */
  KVT_PARSER_DPSK_PGTD = 10,        /* vllm_parse_block_send_multi_tensor_p_gt_d            */
  KVT_PARSER_DPSK_PLTD = 11,        /* vllm_parse_block_send_multi_tensor_p_lt_d            */
  KVT_PARSER_FLASHINFER_PEQD = 12,  /* vllm_parse_flashinfer_block_send_p_eq_d              */
  KVT_PARSER_FLASHINFER_PGTD = 13,  /* vllm_parse_flashinfer_block_send_p_gt_d              */
  KVT_PARSER_HYBRID_FI_PEQD = 14,   /* vllm_parse_qwen3_next_flashinfer_block_send_p_eq_d   */
  KVT_PARSER_HYBRID_FI_PGTD = 15,   /* vllm_parse_qwen3_next_flashinfer_block_send_p_gt_d   */
  KVT_PARSER_HYBRID_FI_PLTD = 16,   /* vllm_parse_qwen3_next_flashinfer_block_send_p_lt_d   */
  KVT_PARSER_KDA_PEQD = 17,         /* parse_kda_block_send_p_eq_d                          */
  KVT_PARSER_KDA_PGTD = 18,         /* parse_kda_block_send_p_gt_d                          */
  KVT_PARSER_KDA_PLTD = 19,         /* parse_kda_block_send_p_lt_d                          */
  KVT_PARSER_KIMI_K3_PEQD = 20,     /* parse_kimi_k3_mla_block_send_p_eq_d                  */
  KVT_PARSER_KIMI_K3_PGTD = 21,     /* parse_kimi_k3_mla_block_send_p_gt_d                  */
  KVT_PARSER_KIMI_K3_PLTD = 22,     /* parse_kimi_k3_mla_block_send_p_lt_d                  */
  KVT_PARSER_TURBOQUANT_PEQD = 23,  /* turboquant_parse_block_send_p_eq_d                   */
  KVT_PARSER_TURBOQUANT_PGTD = 24,  /* turboquant_parse_block_send_p_gt_d                   */
  KVT_PARSER_COUNT = 25
};

/* Error codes. No exception ever crosses the C ABI; the exception classes the
 * reference throws map onto these (kvtransfer/include/parse_block_common.h:64,
 * kvtransfer/src/parse_block_common.cpp:17,28; std::vector::at). */
enum {
  KVT_OK = 0,
  KVT_ERR_OUT_OF_RANGE = 1,  /* std::out_of_range: range/bounds validation, bad block index */
  KVT_ERR_OVERFLOW = 2,      /* std::overflow_error: capacity multiplication overflow       */
  KVT_ERR_INVALID = 3,       /* malformed arguments (null pointers, inconsistent metadata)  */
  KVT_ERR_UNSUPPORTED = 4,   /* std::runtime_error("unsupported cache_shape") and the like  */
  KVT_ERR_HIP = 5,           /* a HIP runtime call failed (see kvt_last_error)              */
  KVT_ERR_NO_DEVICE = 6,     /* GPU entry point called without a usable MI355X              */
  KVT_ERR_TIMEOUT = 7        /* a bounded wait ran out (kvt_session_wait_layer_for)         */
};

/* Per-worker cache geometry consumed by ParseBlock. */
typedef struct kvt_worker_info {
  uint32_t engine_tp_size;
  uint32_t worker_tp_rank;
  uint32_t n_tensors;                       /* entries used in block_sizes / token_sizes */
  uint32_t layer_num_blocks;
  uint64_t block_sizes[KVT_MAX_TENSORS];    /* bytes per block, per cache tensor */
  uint64_t token_sizes[KVT_MAX_TENSORS];    /* bytes per token, per cache tensor */
  uint32_t num_layers;
  uint32_t attn_kernel_blk_ntpb;
  uint32_t indexer_blk_ntpb;
  uint32_t attn_pack_size;
  int32_t  num_kv_heads;                    /* total KV heads of the model; <=0 unknown */
  uint32_t num_gdn_layers;
  uint32_t hybrid_indexer_token_size;
  uint32_t gdn_conv_elem_size;
  uint32_t gdn_ssm_elem_size;
  uint32_t n_conv_state_shape;
  uint64_t conv_state_shape[KVT_MAX_SHAPE_DIMS];
  uint32_t n_ssm_state_shape;
  uint32_t n_gdn_conv_channel_dims;
  uint64_t ssm_state_shape[KVT_MAX_SHAPE_DIMS];
  uint64_t gdn_conv_channel_dims[KVT_MAX_CHANNEL_DIMS];
  uint32_t num_ple_layers;
  uint32_t ple_block_group;
  uint32_t ple_conv_elem_size;
  uint32_t n_ple_conv_state_shape;
  uint64_t ple_conv_state_shape[KVT_MAX_SHAPE_DIMS];
  uint32_t n_ple_conv_channel_dims;
  uint32_t kda_conv_dim_first;              /* bool */
  uint64_t ple_conv_channel_dims[KVT_MAX_CHANNEL_DIMS];
  uint32_t hybrid_attn_token_size;
  uint32_t reserved0;
  uint64_t kda_page_stride;
} kvt_worker_info;

/* One request's contribution to a send step: tokens [seen, seen+new) of the
 * request, the block-id groups on both sides (group g's ids are
 * blocks[group_begin(g) .. +group_len[g]) with group_begin the running sum). */
typedef struct kvt_task {
  uint32_t seen_tokens;
  uint32_t new_tokens;
  uint32_t reach_last_token;                /* bool */
  uint32_t n_src_groups;
  uint32_t n_dst_groups;
  uint32_t reserved0;
  const uint32_t* src_blocks;
  const uint32_t* src_group_len;
  const uint32_t* dst_blocks;
  const uint32_t* dst_group_len;
} kvt_task;

/* Process-wide switches the reference reads from the environment once
 * (kvtransfer/src/envcfg.cpp:327-345). Passed explicitly here. */
typedef struct kvt_parse_opts {
  uint32_t bf16_to_fp8;          /* BLLM_KVTRANS_BF162FP8_CONV (default 0)        */
  uint32_t pad_last_attn_block;  /* BLLM_KVTRANS_PAD_LAST_ATTN_BLOCK (default 1)  */
} kvt_parse_opts;

#ifdef __cplusplus
}
#endif
#endif  /* KVT_TYPES_H_ */
