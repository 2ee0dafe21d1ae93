// Parser compiler: turns one of the reference's 25 ParseBlock functions
// (kvtransfer/src/parse_block_*.cpp), specialised for one sender / receiver
// pair, into a program of layout ops. Every builder cites nothing but
// geometry: the emission order and arithmetic of each op are documented in
// kvt_parse_ops.h and interpreted in kvt_parse.cpp.
#include <algorithm>
#include <limits>

#include "kvt_parse_ops.h"

namespace kvt {
namespace {

u32 popcount16(u32 m) { return static_cast<u32>(__builtin_popcount(m & 0xFFFFu)); }

u64 capacity_of(const kvt_worker_info& w, u32 idx) {
  if (idx >= w.n_tensors || w.layer_num_blocks == 0)
    throw RangeError("KVT parse block capacity metadata mismatch");
  const u64 b = w.block_sizes[idx];
  if (b > std::numeric_limits<u64>::max() / w.layer_num_blocks)
    throw OverflowError("KVT parse block capacity overflow");
  return b * w.layer_num_blocks;
}

void need(bool ok, const char* what) {
  if (!ok) throw InvalidError(std::string("kvt_parser_create: ") + what);
}

struct Builder {
  const kvt_worker_info& s;
  const kvt_worker_info& d;
  u32 valid, tp_size, tp_rank;
  kvt_parse_opts opts;
  kvt_parser* out;

  bool src_rank_valid() const { return (valid >> s.worker_tp_rank) & 1u; }

  void set_lists(u32 n) {
    out->n_lists = n;
    out->caps.assign(std::max<u32>(n, 1), Capacity{0, 0, 1});
  }
  // Capacities are looked up per tensor in emission order; the first failure is
  // remembered and reported by every parse call, as the reference does when
  // make_ipc_block_bounds throws.
  void cap(u32 tensor) {
    if (out->deferred_error != KVT_OK) return;
    try {
      Capacity c;
      c.src = capacity_of(s, tensor);
      c.dst = capacity_of(d, tensor);
      c.scale = opts.bf16_to_fp8 ? 2 : 1;
      if (tensor >= out->caps.size()) out->caps.resize(tensor + 1, Capacity{0, 0, 1});
      out->caps[tensor] = c;
    } catch (const RangeError& e) {
      out->deferred_error = KVT_ERR_OUT_OF_RANGE;
      out->deferred_msg = e.what();
    } catch (const OverflowError& e) {
      out->deferred_error = KVT_ERR_OVERFLOW;
      out->deferred_msg = e.what();
    }
  }

  Op& push(OpKind k, bool only_last = false) {
    out->ops.emplace_back();
    out->ops.back().kind = k;
    out->ops.back().only_last = only_last;
    return out->ops.back();
  }

  // ---- same-geometry walk: one record per block segment
  void walk_same(u32 tensor, u64 B, u64 T) {
    need(T > 0 && B >= T, "token size must be positive and not exceed the block size");
    const u32 ntpb = static_cast<u32>(B / T);
    WalkOp& w = push(OP_WALK).walk;
    w.tensor = tensor;
    w.s.blk_tok = w.s.seg_tok = w.d.blk_tok = w.d.seg_tok = ntpb;
    w.s.blk_bytes = w.d.blk_bytes = B;
    w.s.tok_stride = w.d.tok_stride = T;
    w.unit = T;
  }

  // ---- per-token split between a narrow row (many ranks) and a wide row.
  // `narrow_is_src`: the sender holds the narrow rows (P>D); otherwise P<D.
  WalkOp& walk_split(u32 tensor, u64 nT, u64 nK, u64 wT, u32 ntpb, u64 slot, bool narrow_is_src) {
    need(ntpb > 0, "tokens per block must be positive");
    const u64 k_bytes = opts.bf16_to_fp8 ? nK / 2 : nK;
    WalkOp& w = push(OP_WALK).walk;
    w.tensor = tensor;
    WalkSide narrow, wide;
    narrow.blk_tok = narrow.seg_tok = wide.blk_tok = wide.seg_tok = ntpb;
    narrow.blk_bytes = nT * ntpb;
    narrow.tok_stride = nT;
    wide.blk_bytes = wT * ntpb;
    wide.tok_stride = wT;
    wide.base = slot * k_bytes;
    w.s = narrow_is_src ? narrow : wide;
    w.d = narrow_is_src ? wide : narrow;
    w.per_token = true;
    w.unit = k_bytes;
    return w;
  }

  void ragged_like_split(u32 tensor, const kvt_worker_info& narrow, u32 narrow_tp,
                         const kvt_worker_info& wide, u32 wide_tp, bool narrow_is_src) {
    need(tensor < narrow.n_tensors && tensor < wide.n_tensors, "tensor count mismatch");
    need(wide_tp > 0 && narrow_tp >= wide_tp, "TP sizes do not describe a split");
    const u32 group_n = narrow_tp / wide_tp;
    const u32 slot = narrow.worker_tp_rank % group_n;
    const u64 nT = narrow.token_sizes[tensor], wT = wide.token_sizes[tensor];
    need(nT > 0, "token size must be positive");
    const u32 ntpb = static_cast<u32>(narrow.block_sizes[tensor] / nT);
    const u64 nK = nT / 2, wK = wT / 2;
    WalkOp& w = walk_split(tensor, nT, nK, wT, ntpb, slot, narrow_is_src);
    w.kv = KV_SECOND_PASS;
    w.kv_s_add = narrow_is_src ? nK : wK;
    w.kv_d_add = narrow_is_src ? wK : nK;
    w.pass_len = nK;
  }

  // ---- HND page walk (per head K,V records)
  void walk_hnd(u32 tensor, u32 group, u64 sT, u64 sB, u32 s_ntpb, u32 s_kb, u64 dT, u64 dB,
                u32 d_ntpb, u32 d_kb, u64 row, u32 heads, u64 slot_bytes_on_wide, bool wide_is_dst,
                bool hybrid) {
    need(s_kb > 0 && d_kb > 0 && s_ntpb > 0 && d_ntpb > 0, "tokens per block must be positive");
    WalkOp& w = push(OP_WALK).walk;
    w.tensor = tensor;
    w.s.group = w.d.group = group;
    w.s.blk_tok = s_ntpb;
    w.d.blk_tok = d_ntpb;
    w.s.seg_tok = s_kb;
    w.d.seg_tok = d_kb;
    w.s.blk_bytes = sB;
    w.d.blk_bytes = dB;
    const u64 s_kbs = static_cast<u64>(s_kb) * sT, d_kbs = static_cast<u64>(d_kb) * dT;
    w.s.seg_stride = s_kbs;
    w.d.seg_stride = d_kbs;
    w.s.tok_stride = w.d.tok_stride = row;
    (wide_is_dst ? w.d : w.s).base = slot_bytes_on_wide;
    w.n_loops = 1;
    w.loops[0].count = heads;
    w.loops[0].s_stride = static_cast<u64>(s_kb) * row;
    w.loops[0].d_stride = static_cast<u64>(d_kb) * row;
    w.unit = row;
    w.kv = KV_INTERLEAVED;
    w.kv_s_add = hybrid ? s_kbs / 2 : sB / 2;
    w.kv_d_add = hybrid ? d_kbs / 2 : dB / 2;
  }

  // ---- hybrid NHD attention pages with kernel blocks and layer packing
  void walk_hybrid_attn(u32 group, u64 sT, u64 sB, u32 s_ntpb, u32 s_kb, u64 dT, u64 dB,
                        u32 d_ntpb, u32 d_kb, u32 pack, u64 unit, u64 slot_bytes, bool wide_is_dst) {
    need(s_kb > 0 && d_kb > 0 && pack > 0, "kernel block tokens must be positive");
    need(s_ntpb / pack > 0 && d_ntpb / pack > 0, "tokens per block must be positive");
    WalkOp& w = push(OP_WALK).walk;
    w.s.group = w.d.group = group;
    w.s.blk_tok = pack == 1 ? s_ntpb : s_ntpb / pack;
    w.d.blk_tok = pack == 1 ? d_ntpb : d_ntpb / pack;
    w.s.seg_tok = s_kb;
    w.d.seg_tok = d_kb;
    w.s.blk_bytes = sB;
    w.d.blk_bytes = dB;
    const u64 s_kbs = static_cast<u64>(s_kb) * sT, d_kbs = static_cast<u64>(d_kb) * dT;
    w.s.seg_stride = s_kbs * pack;
    w.d.seg_stride = d_kbs * pack;
    w.s.tok_stride = sT / 2;
    w.d.tok_stride = dT / 2;
    (wide_is_dst ? w.d : w.s).base = slot_bytes;
    w.n_loops = 1;
    w.loops[0].count = pack;
    w.loops[0].s_stride = s_kbs;
    w.loops[0].d_stride = d_kbs;
    w.per_token = true;
    w.unit = unit;
    w.kv = KV_INTERLEAVED;
    w.kv_s_add = s_kbs / 2;
    w.kv_d_add = d_kbs / 2;
  }

  void walk_indexer(u32 group, u64 sB, u64 dB, u32 sn, u32 dn, u32 tok) {
    need(sn > 0 && dn > 0, "indexer tokens per block must be positive");
    // The reference forms the indexer's token term and length as uint32 * uint32
    // (parse_block_qwen3_next.cpp:376-413): for an indexer block of 4 GiB or more they wrap and
    // its ranges point anywhere. Such a geometry is refused here instead of being followed
    // (or silently "corrected" with 64-bit products, which would differ from the reference).
    if (static_cast<u64>(std::max(sn, dn)) * tok > 0xFFFFFFFFull)
      throw OverflowError("KVT parse block: indexer block of 4 GiB or more (tokens per block x "
                          "indexer token size exceeds 32 bits)");
    WalkOp& w = push(OP_WALK).walk;
    w.s.group = w.d.group = group;
    w.s.blk_tok = w.s.seg_tok = sn;
    w.d.blk_tok = w.d.seg_tok = dn;
    w.s.blk_bytes = sB;
    w.d.blk_bytes = dB;
    w.s.tok_stride = w.d.tok_stride = tok;
    w.unit = tok;
  }

  void pages(u32 group, u32 ntpb, u64 page) {
    need(ntpb > 0, "tokens per page must be positive");
    PagesOp& p = push(OP_PAGES).pages;
    p.group = group;
    p.ntpb = ntpb;
    p.page = page;
  }

  void state(u32 first, u32 n, u64 s_page, u64 d_page, u64 len) {
    StateOp& st = push(OP_STATE, true).state;
    st.first_group = first;
    st.n_groups = n;
    st.s_page = s_page;
    st.d_page = d_page;
    st.len = len;
  }

  u64 dim(const u64* v, u32 n, u32 i) const {
    if (i >= n) throw RangeError("state shape metadata too short");
    return v[i];
  }

  // Shape errors of the state metadata surface as out-of-range when the op
  // runs (on the last chunk only), where the reference's .at() throws.
  void gdn_split(u64 sB, u64 dB, u32 gn, u32 goff, bool sender_narrow) {
    const size_t at = out->ops.size();
    push(OP_GDN, true);
    try {
      gdn_split_fill(out->ops[at].gdn, sB, dB, gn, goff, sender_narrow);
    } catch (const RangeError&) {
      out->ops[at].bad_shape = true;
    }
  }

  void gdn_split_fill(GdnOp& g, u64 sB, u64 dB, u32 gn, u32 goff, bool sender_narrow) {
    g.n_groups = s.num_gdn_layers;
    g.s_page = sB;
    g.d_page = dB;
    const u64 e = s.gdn_conv_elem_size;
    g.rows = dim(s.conv_state_shape, s.n_conv_state_shape, 1);
    const u64 row = dim(s.conv_state_shape, s.n_conv_state_shape, 2) * e;
    const u64 conv = g.rows * row;
    const u64 ssm = dim(s.ssm_state_shape, s.n_ssm_state_shape, 1) *
                    dim(s.ssm_state_shape, s.n_ssm_state_shape, 2) *
                    dim(s.ssm_state_shape, s.n_ssm_state_shape, 3) * s.gdn_ssm_elem_size;
    g.s_row = row;
    u64 s_in = 0, d_in = 0;
    if (sender_narrow) {  // P > D: gn sender rows interleave into one receiver row
      g.d_row = gn * row;
      for (u32 c = 0; c < s.n_gdn_conv_channel_dims; ++c) {
        const u64 step = s.gdn_conv_channel_dims[c] * e;
        g.row_pieces.push_back(Piece{s_in, gn * s_in + goff * step, step});
        s_in += step;
      }
      g.ssm = Piece{conv, gn * conv + goff * ssm, ssm};
    } else {  // P < D: this receiver takes its slice of every sender row
      need(gn > 0, "group size must be positive");
      g.d_row = row / gn;
      for (u32 c = 0; c < s.n_gdn_conv_channel_dims; ++c) {
        const u64 ps = s.gdn_conv_channel_dims[c] * e, ds = ps / gn;
        g.row_pieces.push_back(Piece{s_in + goff * ds, d_in, ds});
        s_in += ps;
        d_in += ds;
      }
      g.ssm = Piece{conv + goff * (ssm / gn), g.rows * g.d_row, ssm / gn};
    }
  }

  void ple_split(u64 sB, u64 dB, bool sender_narrow, u32 goff) {
    if (s.num_ple_layers == 0) return;
    if (sender_narrow && goff != 0) return;
    u64 sz = 0;
    bool bad = false;
    try {
      sz = dim(s.ple_conv_state_shape, s.n_ple_conv_state_shape, 1) *
           dim(s.ple_conv_state_shape, s.n_ple_conv_state_shape, 2) * s.ple_conv_elem_size;
    } catch (const RangeError&) {
      bad = true;
    }
    state(s.ple_block_group, s.num_ple_layers, sB, dB, sz);
    out->ops.back().bad_shape = bad;
  }

  // ------------------------------------------------------------ parsers
  void ragged_peqd() {
    need(s.n_tensors >= 1, "source has no cache tensor");
    set_lists(s.n_tensors);
    cap(0);
    walk_same(0, s.block_sizes[0], s.token_sizes[0]);
  }

  void flash_peqd() {
    need(s.n_tensors >= 1, "source has no cache tensor");
    set_lists(s.n_tensors);
    cap(0);
    const u64 kT = s.token_sizes[0] / 2, kB = s.block_sizes[0] / 2;
    walk_same(0, kB, kT);
    WalkOp& w = out->ops.back().walk;
    w.kv = KV_SECOND_PASS;
    w.kv_s_add = kB * s.layer_num_blocks;
    w.kv_d_add = kB * d.layer_num_blocks;
  }

  void flash_pgtd() {
    if (!src_rank_valid()) { out->silent = true; return; }
    need(d.engine_tp_size > 0 && popcount16(valid) >= d.engine_tp_size, "bad TP relation");
    need(s.n_tensors >= 1 && d.n_tensors >= 1, "missing cache tensor");
    const u32 slot = tp_rank % (popcount16(valid) / d.engine_tp_size);
    const u64 pT = s.token_sizes[0], dT = d.token_sizes[0];
    need(pT > 0, "token size must be positive");
    const u64 pK = pT / 2, dK = dT / 2;
    const u32 ntpb = static_cast<u32>(s.block_sizes[0] / pT);
    set_lists(s.n_tensors);
    cap(0);
    WalkOp& w = walk_split(0, pK, pK, dK, ntpb, slot, true);
    w.kv = KV_SECOND_PASS;
    w.kv_s_add = static_cast<u64>(ntpb) * pK * s.layer_num_blocks;
    w.kv_d_add = static_cast<u64>(ntpb) * dK * d.layer_num_blocks;
  }

  void multi_same() {
    set_lists(s.n_tensors);
    for (u32 i = 0; i < s.n_tensors; ++i) {
      cap(i);
      walk_same(i, s.block_sizes[i], s.token_sizes[i]);
      out->ops.back().walk.tensor = i;
    }
  }

  bool same_token_sizes() const {
    if (s.n_tensors != d.n_tensors) return false;
    for (u32 i = 0; i < s.n_tensors; ++i)
      if (s.token_sizes[i] != d.token_sizes[i]) return false;
    return true;
  }

  void multi_split(bool sender_narrow) {
    const kvt_worker_info& narrow = sender_narrow ? s : d;
    const kvt_worker_info& wide = sender_narrow ? d : s;
    const u32 narrow_tp = sender_narrow ? tp_size : d.engine_tp_size;
    const u32 wide_tp = sender_narrow ? d.engine_tp_size : tp_size;
    set_lists(narrow.n_tensors);
    for (u32 c = 0; c < narrow.n_tensors; ++c) {
      cap(c);
      ragged_like_split(c, narrow, narrow_tp, wide, wide_tp, sender_narrow);
    }
  }

  int fi_heads() const {
    if (s.num_kv_heads > 0 && static_cast<u32>(s.num_kv_heads) >= s.engine_tp_size)
      return s.num_kv_heads / static_cast<int>(s.engine_tp_size);
    return std::max(1, s.num_kv_heads);
  }

  void flashinfer(bool gt) {
    u32 slot = 0;
    if (gt) {
      if (!src_rank_valid()) { out->silent = true; return; }
      need(d.engine_tp_size > 0 && popcount16(valid) >= d.engine_tp_size, "bad TP relation");
      slot = tp_rank % (popcount16(valid) / d.engine_tp_size);
    }
    need(s.n_tensors >= 1 && d.n_tensors >= 1, "missing cache tensor");
    const u64 pT = s.token_sizes[0], pB = s.block_sizes[0], dB = d.block_sizes[0];
    need(pT > 0, "token size must be positive");
    const u32 ntpb = static_cast<u32>(pB / pT);
    const u32 heads = static_cast<u32>(fi_heads());
    const u64 row = pT / 2 / heads;
    set_lists(1);
    cap(0);
    walk_hnd(0, 0, pT, pB, ntpb, ntpb, d.token_sizes[0], dB, ntpb, ntpb, row, heads,
             static_cast<u64>(slot) * heads * ntpb * row, true, false);
  }

  struct Hybrid {
    u64 pT, pB, dT, dB;
    u32 s_ntpb, d_ntpb, pack;
  };

  Hybrid hybrid_geometry() {
    need(s.n_tensors >= 1 && d.n_tensors >= 1, "missing cache tensor");
    Hybrid h;
    h.pT = s.token_sizes[0];
    h.pB = s.block_sizes[0];
    h.dT = d.token_sizes[0];
    h.dB = d.block_sizes[0];
    need(h.pT > 0 && h.dT > 0, "token size must be positive");
    h.s_ntpb = static_cast<u32>(h.pB / h.pT);
    h.d_ntpb = static_cast<u32>(h.dB / h.dT);
    h.pack = s.attn_pack_size == 0 ? 1u : s.attn_pack_size;
    return h;
  }

  void hybrid_peqd(bool hnd) {
    const Hybrid h = hybrid_geometry();
    set_lists(s.n_tensors);
    cap(0);
    u32 g = s.num_gdn_layers;
    if (s.indexer_blk_ntpb > 0) pages(g++, s.indexer_blk_ntpb, h.pB);
    const u64 attn_ntpb = hnd ? h.s_ntpb : h.pB / h.pT / h.pack;
    pages(g, static_cast<u32>(attn_ntpb), h.pB);
    state(0, s.num_gdn_layers, h.pB, h.pB, h.pB);
    if (s.num_ple_layers > 0) state(s.ple_block_group, s.num_ple_layers, h.pB, h.pB, h.pB);
  }

  void fill(FillKind kind, u32 group, const Hybrid& h, u64 sB, u64 dB, u32 d_blk_tok, u32 s_kb,
            u32 d_kb, u64 d_seg_bytes, u64 d_tok_stride, u64 unit, u64 d_base, u64 d_half,
            u32 heads, u64 d_head_stride) {
    need(d_blk_tok > 0 && s_kb > 0 && d_kb > 0, "tokens per block must be positive");
    // the fills emit one record per token of a block
    need(d_blk_tok <= (1u << 16), "more than 65536 tokens per block");
    FillOp& f = push(OP_FILL, true).fill;
    f.kind = kind;
    f.group = group;
    f.s_page = sB;
    f.d_page = dB;
    f.d_blk_tok = d_blk_tok;
    f.s_seg_tok = s_kb;
    f.d_seg_tok = d_kb;
    f.pack = h.pack;
    f.d_seg_bytes = d_seg_bytes;
    f.d_tok_stride = d_tok_stride;
    f.unit = unit;
    f.d_base = d_base;
    f.d_half = d_half;
    f.heads = heads;
    f.d_head_stride = d_head_stride;
  }

  void hybrid_pgtd(bool hnd) {
    need(d.engine_tp_size > 0 && s.engine_tp_size >= d.engine_tp_size, "bad TP relation");
    const u32 gdn_n = s.engine_tp_size / d.engine_tp_size;
    const u32 gdn_off = s.worker_tp_rank % gdn_n;
    const u32 attn_n = popcount16(valid) / d.engine_tp_size;
    need(hnd || attn_n > 0, "no valid sender rank per receiver");
    const u32 attn_off = attn_n > 0 ? tp_rank % attn_n : 0;
    Hybrid h = hybrid_geometry();
    set_lists(s.n_tensors);
    cap(0);
    // the NHD variant re-derives the page sizes from the token sizes
    const u64 pB = hnd ? h.pB : h.pT * h.s_ntpb, dB = hnd ? h.dB : h.dT * h.d_ntpb;
    gdn_split(pB, dB, gdn_n, gdn_off, true);
    ple_split(pB, dB, true, gdn_off);
    u32 g = s.num_gdn_layers;
    if (s.indexer_blk_ntpb > 0 && d.indexer_blk_ntpb > 0) {
      if (s.worker_tp_rank % gdn_n == 0)
        walk_indexer(g, pB, dB, s.indexer_blk_ntpb, d.indexer_blk_ntpb,
                     s.hybrid_indexer_token_size);
      g += 1;
    }
    if (!src_rank_valid()) return;
    const u32 s_kb = s.attn_kernel_blk_ntpb, d_kb = d.attn_kernel_blk_ntpb;
    if (hnd) {
      const u32 heads = static_cast<u32>(
          std::max(1, s.num_kv_heads / static_cast<int>(s.engine_tp_size)));
      const u64 row = h.pT / 2 / heads;
      const u64 slot = static_cast<u64>(attn_off) * heads * d_kb * row;
      walk_hnd(0, g, h.pT, pB, h.s_ntpb, s_kb, h.dT, dB, h.d_ntpb, d_kb, row, heads, slot, true,
               true);
      if (opts.pad_last_attn_block)
        fill(FILL_HND_LAST, g, h, pB, dB, h.d_ntpb, 1, 1, 0, 0, row,
             static_cast<u64>(attn_off) * heads * h.d_ntpb * row,
             static_cast<u64>(h.d_ntpb) * h.dT / 2, heads, static_cast<u64>(h.d_ntpb) * row);
    } else {
      const u64 ps = h.pT / 2;
      walk_hybrid_attn(g, h.pT, pB, h.s_ntpb, s_kb, h.dT, dB, h.d_ntpb, d_kb, h.pack, ps,
                       attn_off * ps, true);
      if (opts.pad_last_attn_block) {
        const u64 d_kbs = static_cast<u64>(d_kb) * h.dT;
        fill(FILL_ATTN_LAST, g, h, pB, dB, h.pack == 1 ? h.d_ntpb : h.d_ntpb / h.pack, s_kb, d_kb,
             d_kbs, h.dT / 2, ps, attn_off * ps, d_kbs / 2, 1, 0);
      }
    }
  }

  void hybrid_pltd(bool hnd) {
    const u32 p_tp = s.engine_tp_size, d_tp = d.engine_tp_size;
    need(p_tp > 0 && d_tp >= p_tp, "bad TP relation");
    const u32 gdn_n = d_tp / p_tp;
    const u32 gdn_off = d.worker_tp_rank % gdn_n;
    const Hybrid h = hybrid_geometry();
    set_lists(s.n_tensors);
    cap(0);
    u32 g = s.num_gdn_layers;
    const u32 p_in = s.indexer_blk_ntpb, d_in = d.indexer_blk_ntpb;
    if (h.pT == h.dT) {
      if (p_in > 0) pages(g++, p_in, h.pB);
      pages(g, hnd ? h.s_ntpb : static_cast<u32>(h.pB / h.pT / h.pack), h.pB);
    } else {
      const u32 attn_n = static_cast<u32>(h.pT / h.dT);
      need(attn_n > 0 && d_tp / (p_tp * attn_n) > 0, "token sizes do not describe a split");
      const u32 replicas = d_tp / (p_tp * attn_n);
      const u32 attn_off = (d.worker_tp_rank / replicas) % attn_n;
      if (p_in > 0) walk_indexer(g++, h.pB, h.dB, p_in, d_in, s.hybrid_indexer_token_size);
      const u32 s_kb = s.attn_kernel_blk_ntpb, d_kb = d.attn_kernel_blk_ntpb;
      if (hnd) {
        const int total = s.num_kv_heads;
        const u32 d_heads = static_cast<u32>(total) >= d_tp ? static_cast<u32>(total) / d_tp : 1u;
        const u64 row = h.dT / 2 / d_heads;
        // the sender's (wide) page holds attn_n receivers' head sections
        walk_hnd(0, g, h.pT, h.pB, h.s_ntpb, s_kb, h.dT, h.dB, h.d_ntpb, d_kb, row, d_heads,
                 static_cast<u64>(attn_off) * d_heads * s_kb * row, false, true);
        if (opts.pad_last_attn_block)
          fill(FILL_HND_TAIL, g, h, h.pB, h.dB, h.d_ntpb, 1, h.d_ntpb, 0, row, row, 0, h.dB / 2,
               d_heads, static_cast<u64>(h.d_ntpb) * row);
      } else {
        const u64 ds = h.dT / 2;
        walk_hybrid_attn(g, h.pT, h.pB, h.s_ntpb, s_kb, h.dT, h.dB, h.d_ntpb, d_kb, h.pack, ds,
                         attn_off * ds, false);
        if (opts.pad_last_attn_block) {
          const u64 d_kbs = static_cast<u64>(d_kb) * h.dT;
          fill(FILL_ATTN_TAIL, g, h, h.pB, h.dB, h.pack == 1 ? h.d_ntpb : h.d_ntpb / h.pack, 1,
               d_kb, d_kbs, ds, ds, 0, d_kbs / 2, 1, 0);
        }
      }
    }
    gdn_split(h.pB, h.dB, gdn_n, gdn_off, false);
    ple_split(h.pB, h.dB, false, gdn_off);
  }

  // ---- KDA state pages ([conv][recurrent][padding], SD or DS conv layout)
  u64 kda_stride(const kvt_worker_info& w) const {
    if (w.kda_page_stride != 0) return w.kda_page_stride;
    if (w.n_tensors < 1) throw RangeError("no cache tensor registered");
    return w.block_sizes[0];
  }

  // rel: 0 P==D, +1 P>D, -1 P<D. The page stride is looked up before the
  // "last chunk only" gate for P==D and after it otherwise (a missing tensor is
  // then reported on the last chunk only), as the reference orders it.
  void kda_state(int rel) {
    set_lists(1);
    if (rel == 0) {
      const u64 sp = kda_stride(s), dp = kda_stride(d);
      cap(0);
      state(0, s.num_gdn_layers, sp, dp, sp);
      return;
    }
    need(s.engine_tp_size > 0 && d.engine_tp_size > 0, "bad TP relation");
    const u32 gn = rel > 0 ? s.engine_tp_size / d.engine_tp_size : d.engine_tp_size / s.engine_tp_size;
    need(gn > 0, "bad TP relation");
    const u32 goff = (rel > 0 ? s.worker_tp_rank : d.worker_tp_rank) % gn;
    const size_t at = out->ops.size();
    push(OP_GDN, true);
    try {
      GdnOp& g = out->ops[at].gdn;
      g.n_groups = s.num_gdn_layers;
      g.s_page = kda_stride(s);
      g.d_page = kda_stride(d);
      const u64 e = s.gdn_conv_elem_size;
      const bool ds = s.kda_conv_dim_first != 0;
      const u64 state_len = dim(s.conv_state_shape, s.n_conv_state_shape, ds ? 2 : 1);
      const u64 qkv = dim(s.conv_state_shape, s.n_conv_state_shape, ds ? 1 : 2);
      const u64 conv = state_len * qkv * e;
      const u64 rec = dim(s.ssm_state_shape, s.n_ssm_state_shape, 1) *
                      dim(s.ssm_state_shape, s.n_ssm_state_shape, 2) *
                      dim(s.ssm_state_shape, s.n_ssm_state_shape, 3) * s.gdn_ssm_elem_size;
      // DS keeps each channel's history contiguous: one "row" whose pieces are whole
      // components; SD repeats the q/k/v placement for every history row.
      g.rows = ds ? 1 : state_len;
      const u64 per_piece = ds ? state_len * e : e;
      g.s_row = qkv * e;
      u64 s_in = 0, d_in = 0;
      if (rel > 0) {
        g.d_row = gn * g.s_row;
        for (u32 c = 0; c < s.n_gdn_conv_channel_dims; ++c) {
          const u64 comp = s.gdn_conv_channel_dims[c] * per_piece;
          g.row_pieces.push_back(Piece{s_in, gn * s_in + goff * comp, comp});
          s_in += comp;
        }
        g.ssm = Piece{conv, gn * conv + goff * rec, rec};
      } else {
        g.d_row = g.s_row / gn;
        for (u32 c = 0; c < s.n_gdn_conv_channel_dims; ++c) {
          const u64 comp = (s.gdn_conv_channel_dims[c] / gn) * per_piece;
          g.row_pieces.push_back(Piece{s_in + goff * comp, d_in, comp});
          s_in += gn * comp;
          d_in += comp;
        }
        g.ssm = Piece{conv + goff * (rec / gn), ds ? d_in : conv / gn, rec / gn};
      }
    } catch (const RangeError&) {
      out->ops[at].bad_shape = true;
    }
    cap(0);
  }

  void kimi_mla() {
    if (!src_rank_valid()) return;
    const size_t at = out->ops.size();
    MlaOp& m = push(OP_MLA).mla;
    m.group = s.num_gdn_layers;
    if (s.n_tensors < 1 || d.n_tensors < 1) {
      out->ops[at].bad_shape = true;
      return;
    }
    need(s.token_sizes[0] > 0 && d.token_sizes[0] > 0, "token size must be positive");
    m.s_mgr_tok = static_cast<u32>(s.block_sizes[0] / s.token_sizes[0]);
    m.d_mgr_tok = static_cast<u32>(d.block_sizes[0] / d.token_sizes[0]);
    m.kernel_tok = s.attn_kernel_blk_ntpb;
    need(m.s_mgr_tok > 0 && m.d_mgr_tok > 0 && m.kernel_tok > 0, "tokens per block must be positive");
    m.tok_bytes = s.hybrid_attn_token_size;
    m.kernel_bytes = static_cast<u64>(m.kernel_tok) * m.tok_bytes;
    m.s_page = s.kda_page_stride != 0 ? s.kda_page_stride : s.block_sizes[0];
    m.d_page = d.kda_page_stride != 0 ? d.kda_page_stride : d.block_sizes[0];
    m.equal_tp = s.engine_tp_size == d.engine_tp_size;
    m.pad = opts.pad_last_attn_block != 0;
    set_lists(1);
    cap(0);
  }

  void build(int parser_id) {
    switch (parser_id) {
      case KVT_PARSER_RAGGED_PEQD: ragged_peqd(); break;
      case KVT_PARSER_RAGGED_PGTD_DPSK:
        if (s.worker_tp_rank != 0) { out->silent = true; break; }
        ragged_peqd();
        break;
      case KVT_PARSER_RAGGED_PGTD:
        need(s.n_tensors >= 1, "source has no cache tensor");
        set_lists(s.n_tensors);
        cap(0);
        ragged_like_split(0, s, tp_size, d, d.engine_tp_size, true);
        break;
      case KVT_PARSER_RAGGED_PLTD:
        need(d.n_tensors >= 1, "destination has no cache tensor");
        set_lists(d.n_tensors);
        cap(0);
        ragged_like_split(0, d, d.engine_tp_size, s, tp_size, false);
        break;
      case KVT_PARSER_FLASH_PEQD: flash_peqd(); break;
      case KVT_PARSER_FLASH_PGTD: flash_pgtd(); break;
      case KVT_PARSER_DPSK_PEQD:
        if (!src_rank_valid()) { out->silent = true; break; }
        multi_same();
        break;
      case KVT_PARSER_DPSK_PGTD:
        if (same_token_sizes()) {
          if (s.worker_tp_rank != 0) { out->silent = true; break; }
          multi_same();
        } else {
          multi_split(true);
        }
        break;
      case KVT_PARSER_DPSK_PLTD: multi_split(false); break;
      case KVT_PARSER_FLASHINFER_PEQD: flashinfer(false); break;
      case KVT_PARSER_FLASHINFER_PGTD: flashinfer(true); break;
      case KVT_PARSER_TURBOQUANT_PEQD:
      case KVT_PARSER_HYBRID_PEQD: hybrid_peqd(false); break;
      case KVT_PARSER_TURBOQUANT_PGTD:
      case KVT_PARSER_HYBRID_PGTD: hybrid_pgtd(false); break;
      case KVT_PARSER_HYBRID_PLTD: hybrid_pltd(false); break;
      case KVT_PARSER_HYBRID_FI_PEQD: hybrid_peqd(true); break;
      case KVT_PARSER_HYBRID_FI_PGTD: hybrid_pgtd(true); break;
      case KVT_PARSER_HYBRID_FI_PLTD: hybrid_pltd(true); break;
      case KVT_PARSER_KDA_PEQD: kda_state(0); break;
      case KVT_PARSER_KDA_PGTD: kda_state(1); break;
      case KVT_PARSER_KDA_PLTD: kda_state(-1); break;
      case KVT_PARSER_KIMI_K3_PEQD: kimi_mla(); kda_state(0); break;
      case KVT_PARSER_KIMI_K3_PGTD: kimi_mla(); kda_state(1); break;
      case KVT_PARSER_KIMI_K3_PLTD: kimi_mla(); kda_state(-1); break;
      default:
        throw InvalidError("parser id not supported by this build");
    }
  }
};

}  // namespace

void build_parser(int parser_id, const kvt_worker_info& src, const kvt_worker_info& dst,
                  uint32_t valid_mask, uint32_t kvt_tp_size, uint32_t kvt_tp_rank,
                  const kvt_parse_opts& opts, kvt_parser* out) {
  Builder b{src, dst, valid_mask, kvt_tp_size, kvt_tp_rank, opts, out};
  b.build(parser_id);
}

}  // namespace kvt
