// The compiled form of a parser: a short program of layout ops that
// kvt_parse_block() interprets for every task (shared by the compiler in
// kvt_parse_build.cpp and the interpreter in kvt_parse.cpp).
#ifndef KVT_PARSE_OPS_H_
#define KVT_PARSE_OPS_H_

#include <string>
#include <vector>

#include "kvt_internal.h"

namespace kvt {

typedef uint64_t u64;
typedef uint32_t u32;

struct Capacity {
  u64 src, dst, scale;
};

// One side (sender or receiver) of a token walk: how a token position maps to
// a byte offset inside that side's layer tensor.
struct WalkSide {
  u32 group = 0;       // block-id group of the task to index
  u32 blk_tok = 1;     // tokens addressed by one block id
  u32 seg_tok = 1;     // tokens per contiguous segment (kernel block)
  u64 blk_bytes = 0;   // bytes between consecutive block ids
  u64 seg_stride = 0;  // bytes between consecutive segments inside a block
  u64 tok_stride = 0;  // bytes between consecutive tokens inside a segment
  u64 base = 0;        // constant byte offset (e.g. this rank's slot in a wider row)
};

struct Loop {
  u32 count = 1;
  u64 s_stride = 0, d_stride = 0;
};

enum KvMode { KV_NONE, KV_INTERLEAVED, KV_SECOND_PASS };

// Token walk: positions [seen, seen+new) are cut into segments bounded by both
// sides' seg_tok; each segment emits  loops[0] x loops[1] x (tokens) x (K,V).
struct WalkOp {
  u32 tensor = 0;
  WalkSide s, d;
  u32 n_loops = 0;
  Loop loops[2];
  bool per_token = false;  // one record per token (length = unit) vs per segment (k * unit)
  u64 unit = 0;
  KvMode kv = KV_NONE;
  u64 kv_s_add = 0, kv_d_add = 0;
  u64 pass_len = 0;        // KV_SECOND_PASS: 0 = same length as the first-pass record
};

// Whole-page walk of a block group (pages sent only once complete).
struct PagesOp {
  u32 tensor = 0, group = 0, ntpb = 1;
  u64 page = 0;
};

// `len` bytes from the start of every page of `n_groups` consecutive groups.
struct StateOp {
  u32 tensor = 0, first_group = 0, n_groups = 0;
  u64 s_page = 0, d_page = 0, len = 0;
};

struct Piece {
  u64 s_off, d_off, len;
};

// Linear-attention state page split between TP ranks: per conv row a few
// channel pieces, then one recurrent-state piece.
struct GdnOp {
  u32 tensor = 0, n_groups = 0;
  u64 s_page = 0, d_page = 0;
  u64 rows = 0, s_row = 0, d_row = 0;
  std::vector<Piece> row_pieces;
  Piece ssm{0, 0, 0};
};

enum FillKind { FILL_ATTN_LAST, FILL_ATTN_TAIL, FILL_HND_LAST, FILL_HND_TAIL };

// Zero fill of not-yet-written destination token slots from the request's
// first source page (kept all-zero by the engine).
struct FillOp {
  FillKind kind = FILL_ATTN_LAST;
  u32 tensor = 0, group = 0;
  u64 s_page = 0, d_page = 0;   // page strides
  u32 d_blk_tok = 1;            // per-layer tokens per destination block id
  u32 s_seg_tok = 1, d_seg_tok = 1;
  u32 pack = 1;
  u64 d_seg_bytes = 0;          // bytes of one destination kernel block
  u64 d_tok_stride = 0;         // K (or V) bytes per destination token
  u64 unit = 0;                 // bytes per filled token record / per token of a run
  u64 d_base = 0;
  u64 d_half = 0;               // K -> V distance inside a kernel block / page
  u32 heads = 1;
  u64 d_head_stride = 0;
};

// Real MLA prefix of KDA-sized physical pages (Kimi-K3): whole manager blocks
// when both sides use the same TP, kernel pages plus a zero-filled tail otherwise.
struct MlaOp {
  u32 group = 0;
  bool equal_tp = true, pad = true;
  u32 s_mgr_tok = 1, d_mgr_tok = 1, kernel_tok = 1;
  u64 s_page = 0, d_page = 0, kernel_bytes = 0, tok_bytes = 0;
};

enum OpKind { OP_WALK, OP_PAGES, OP_STATE, OP_GDN, OP_FILL, OP_MLA };

struct Op {
  OpKind kind;
  bool only_last = false;
  bool bad_shape = false;  // state-shape metadata too short: running the op is an error
  WalkOp walk;
  PagesOp pages;
  StateOp state;
  GdnOp gdn;
  FillOp fill;
  MlaOp mla;
};

// Compiles the reference parser `parser_id` for one (sender, receiver) pair into `out`.
// Throws InvalidError for metadata no parser can work with.
void build_parser(int parser_id, const kvt_worker_info& src, const kvt_worker_info& dst,
                  uint32_t valid_mask, uint32_t kvt_tp_size, uint32_t kvt_tp_rank,
                  const kvt_parse_opts& opts, kvt_parser* out);

}  // namespace kvt

struct kvt_parser {
  bool silent = false;              // this rank sends nothing and leaves the lists untouched
  uint32_t n_lists = 0;             // outer size the lists are resized to
  int deferred_error = KVT_OK;      // capacity error raised on every parse call
  std::string deferred_msg;
  std::vector<kvt::Capacity> caps;  // per tensor
  std::vector<kvt::Op> ops;
};

#endif  // KVT_PARSE_OPS_H_
