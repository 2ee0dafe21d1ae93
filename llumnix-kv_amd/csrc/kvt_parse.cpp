// Layout-aware block-table parsing (host side).
//
// The reference implements ParseBlock as ~25 hand-written functions, one per
// (cache shape x TP relation), each re-deriving its strides on every call
// (kvtransfer/src/parse_block_*.cpp). Here a parser is *compiled once per
// destination* into a short program of layout ops -- token walks with a strided
// record nest, whole-page walks, state-page copies, GDN conv/ssm splits and
// zero fills -- and kvt_parse_block() merely interprets that program for a
// task. The emitted (src_offset, dst_offset, length) sequence is identical,
// record for record, to what the corresponding reference function appends.
//
// An arithmetic note: the reference forms a few products in 32 bits. The kernel-block index
// times the pack size never exceeds the tokens per block, a 32-bit number, so 64-bit
// arithmetic gives the same value; the indexer's token term and length (tokens x indexer token
// size) wrap in the reference for indexer blocks of 4 GiB or more, and kvt_parser_create
// refuses such a geometry with KVT_ERR_OVERFLOW rather than following or "correcting" it.
#include <algorithm>
#include <cstring>
#include <limits>
#include <memory>

#include "kvt_parse_ops.h"

namespace kvt {
namespace {

// ------------------------------------------------------------------ interpreter

struct Groups {
  const u32* ids;
  const u32* lens;
  u32 n;
  // -> (pointer, length) of group g; throws like std::vector::at
  void get(u32 g, const u32*& p, u64& len) const {
    if (g >= n) throw RangeError("block group index out of range");
    u64 pos = 0;
    for (u32 i = 0; i < g; ++i) pos += lens[i];
    p = ids + pos;
    len = lens[g];
  }
};

struct Sink {
  RunList* out;
  Capacity cap;
  std::vector<kvt_run>* runs = nullptr;  // run form: every record becomes (part of) a kvt_run

  void check(u64 so, u64 dof, u64 len) const {
    const u64 M = std::numeric_limits<u64>::max();
    const bool ovf = cap.scale == 0 || len > M / cap.scale;
    const u64 eff = ovf ? M : len * cap.scale;
    if (len == 0 || ovf || so > cap.src || eff > cap.src - so || dof > cap.dst ||
        len > cap.dst - dof)
      throw RangeError("KVT GPU buffer range validation failed");
  }
  void put(u64 so, u64 dof, u64 len) {
    check(so, dof, len);
    if (runs) {
      kvt_run r{};
      r.src_offset = so;
      r.dst_offset = dof;
      r.length = len;
      r.n[0] = r.n[1] = r.n[2] = 1;
      runs->push_back(r);
    } else {
      out->push_back(kvt_ipc_block{so, dof, len});
    }
  }
  // Run form only. Offsets grow with every index, so the nest is inside the
  // buffers exactly when its last range is (an index product that overflows
  // 64 bits cannot be inside any buffer).
  void put_nest(kvt_run r) {
    u64 s_max = r.src_offset, d_max = r.dst_offset;
    for (int k = 0; k < 3; ++k) {
      const u64 steps = r.n[k] - 1;
      u64 ds, dd;
      if (__builtin_mul_overflow(steps, r.src_stride[k], &ds) ||
          __builtin_add_overflow(s_max, ds, &s_max) ||
          __builtin_mul_overflow(steps, r.dst_stride[k], &dd) ||
          __builtin_add_overflow(d_max, dd, &d_max))
        throw RangeError("KVT GPU buffer range validation failed");
    }
    check(r.src_offset, r.dst_offset, r.length);
    check(s_max, d_max, r.length);
    runs->push_back(r);
  }
  size_t size() const { return runs ? runs->size() : out->size(); }
};

inline u32 id_at(const u32* p, u64 n, u64 i) {
  if (i >= n) throw RangeError("block index out of range");
  return p[i];
}

inline u64 side_offset(const WalkSide& w, u32 pos, const u32* ids, u64 n_ids) {
  const u32 bi = pos / w.blk_tok;
  return static_cast<u64>(id_at(ids, n_ids, bi)) * w.blk_bytes +
         static_cast<u64>((pos % w.blk_tok) / w.seg_tok) * w.seg_stride +
         static_cast<u64>(pos % w.seg_tok) * w.tok_stride + w.base;
}

void run_walk(const WalkOp& w, const kvt_task& t, const Groups& sg, const Groups& dg, Sink& sink) {
  const u32 *sid, *did;
  u64 sn, dn;
  sg.get(w.s.group, sid, sn);
  dg.get(w.d.group, did, dn);
  const size_t first = sink.size();
  u32 pos = t.seen_tokens, rem = t.new_tokens;
  const u32 c0 = w.n_loops > 0 ? w.loops[0].count : 1;
  const u32 c1 = w.n_loops > 1 ? w.loops[1].count : 1;
  while (rem > 0) {
    const u32 k = std::min(std::min(w.s.seg_tok - pos % w.s.seg_tok, w.d.seg_tok - pos % w.d.seg_tok), rem);
    const u64 so = side_offset(w.s, pos, sid, sn);
    const u64 dof = side_offset(w.d, pos, did, dn);
    const u32 n_tok = w.per_token ? k : 1;
    const u64 len = w.per_token ? w.unit : static_cast<u64>(k) * w.unit;
    if (sink.runs && c1 == 1) {  // the whole segment in closed form: loop x tokens x (K, V)
      kvt_run r{};
      r.src_offset = so;
      r.dst_offset = dof;
      r.length = len;
      r.n[0] = c0;
      r.src_stride[0] = c0 > 1 ? w.loops[0].s_stride : 0;
      r.dst_stride[0] = c0 > 1 ? w.loops[0].d_stride : 0;
      r.n[1] = n_tok;
      r.src_stride[1] = n_tok > 1 ? w.s.tok_stride : 0;
      r.dst_stride[1] = n_tok > 1 ? w.d.tok_stride : 0;
      r.n[2] = w.kv == KV_INTERLEAVED ? 2 : 1;
      r.src_stride[2] = w.kv == KV_INTERLEAVED ? w.kv_s_add : 0;
      r.dst_stride[2] = w.kv == KV_INTERLEAVED ? w.kv_d_add : 0;
      sink.put_nest(r);
    } else {
      for (u32 a = 0; a < c0; ++a)
        for (u32 b = 0; b < c1; ++b) {
          const u64 s1 = so + a * w.loops[0].s_stride + b * w.loops[1].s_stride;
          const u64 d1 = dof + a * w.loops[0].d_stride + b * w.loops[1].d_stride;
          for (u32 i = 0; i < n_tok; ++i) {
            const u64 s2 = s1 + i * w.s.tok_stride, d2 = d1 + i * w.d.tok_stride;
            sink.put(s2, d2, len);
            if (w.kv == KV_INTERLEAVED) sink.put(s2 + w.kv_s_add, d2 + w.kv_d_add, len);
          }
        }
    }
    pos += k;
    rem -= k;
  }
  if (w.kv == KV_SECOND_PASS) {
    const size_t last = sink.size();
    for (size_t i = first; i < last; ++i) {
      if (sink.runs) {
        kvt_run r = (*sink.runs)[i];
        r.src_offset += w.kv_s_add;
        r.dst_offset += w.kv_d_add;
        if (w.pass_len) r.length = w.pass_len;
        sink.put_nest(r);
      } else {
        const kvt_ipc_block k = (*sink.out)[i];
        sink.put(k.src_offset + w.kv_s_add, k.dst_offset + w.kv_d_add,
                 w.pass_len ? w.pass_len : k.length);
      }
    }
  }
}

void run_pages(const PagesOp& p, const kvt_task& t, const Groups& sg, const Groups& dg,
               Sink& sink) {
  const u32 *sid, *did;
  u64 sn, dn;
  sg.get(p.group, sid, sn);
  dg.get(p.group, did, dn);
  const bool last = t.reach_last_token != 0;
  u32 pos = t.seen_tokens, rem = t.new_tokens;
  while (rem > 0) {
    const u32 bi = pos / p.ntpb, ti = pos % p.ntpb;
    const u64 so = static_cast<u64>(id_at(sid, sn, bi)) * p.page;
    const u64 dof = static_cast<u64>(id_at(did, dn, bi)) * p.page;
    const u32 k = std::min(p.ntpb - ti, rem);
    // a page goes out when it is complete after this chunk, or the request ends
    const bool send = k == p.ntpb || last || (ti != 0 && ti + k == p.ntpb);
    if (send) sink.put(so, dof, p.page);
    pos += k;
    rem -= k;
  }
  if (last) {  // blocks allocated beyond the last token (kept zero by the engine)
    const u64 next = (static_cast<u64>(pos) + p.ntpb - 1) / p.ntpb;
    for (u64 i = next; i < sn; ++i)
      sink.put(static_cast<u64>(sid[i]) * p.page, static_cast<u64>(id_at(did, dn, i)) * p.page,
               p.page);
  }
}

void run_state(const StateOp& st, const Groups& sg, const Groups& dg, Sink& sink) {
  for (u32 g = 0; g < st.n_groups; ++g) {
    const u32 *sid, *did;
    u64 sn, dn;
    sg.get(st.first_group + g, sid, sn);
    dg.get(st.first_group + g, did, dn);
    for (u64 i = 0; i < sn; ++i)
      sink.put(static_cast<u64>(sid[i]) * st.s_page, static_cast<u64>(id_at(did, dn, i)) * st.d_page,
               st.len);
  }
}

void run_gdn(const GdnOp& g, const Groups& sg, const Groups& dg, Sink& sink) {
  // conv rows = convolution width - 1 (a handful); the trip count below comes straight from
  // caller metadata, so refuse values that can only be garbage instead of spinning on them
  if (g.rows > (1u << 16)) throw RangeError("state shape metadata implausible: conv rows");
  for (u32 grp = 0; grp < g.n_groups; ++grp) {
    const u32 *sid, *did;
    u64 sn, dn;
    sg.get(grp, sid, sn);
    dg.get(grp, did, dn);
    for (u64 i = 0; i < sn; ++i) {
      const u64 so = static_cast<u64>(sid[i]) * g.s_page;
      const u64 dof = static_cast<u64>(id_at(did, dn, i)) * g.d_page;
      for (u64 r = 0; r < g.rows; ++r)
        for (const Piece& p : g.row_pieces)
          sink.put(so + r * g.s_row + p.s_off, dof + r * g.d_row + p.d_off, p.len);
      sink.put(so + g.ssm.s_off, dof + g.ssm.d_off, g.ssm.len);
    }
  }
}

void zero_run(Sink& sink, u64 zero_src, u64 dof, u64 len, u64 max_piece) {
  // A fill is cut into pieces no longer than the (all-zero) source page. Real geometries need
  // a handful of pieces; a page of a few bytes against a huge fill is malformed metadata and
  // would otherwise emit billions of ranges.
  if (max_piece == 0 || len / max_piece > (1u << 20))
    throw RangeError("zero fill: source page too small for the range to fill");
  for (u64 done = 0; done < len;) {
    const u64 n = std::min(max_piece, len - done);
    sink.put(zero_src, dof + done, n);
    done += n;
  }
}

void run_fill(const FillOp& f, const kvt_task& t, const Groups& sg, const Groups& dg, Sink& sink) {
  const u32 *sid, *did;
  u64 sn, dn;
  sg.get(f.group, sid, sn);
  dg.get(f.group, did, dn);
  const u32 total = t.seen_tokens + t.new_tokens;
  switch (f.kind) {
    case FILL_ATTN_LAST: {  // rest of the last, partly written destination block; token records
      if (total == 0) return;
      const u32 filled = total % f.d_blk_tok;
      if (filled == 0) return;
      u32 todo = f.d_blk_tok - filled;
      const u64 zero = static_cast<u64>(id_at(sid, sn, 0)) * f.s_page;
      u32 dpos = total, spos = 0;
      while (todo > 0) {
        const u32 dbi = dpos / f.d_blk_tok;
        const u64 seg = static_cast<u64>((dpos % f.d_blk_tok) / f.d_seg_tok) * f.pack * f.d_seg_bytes;
        const u32 dt0 = dpos % f.d_seg_tok, st0 = spos % f.s_seg_tok;
        const u64 dof = static_cast<u64>(id_at(did, dn, dbi)) * f.d_page;
        const u32 k = std::min(std::min(f.s_seg_tok - st0, f.d_seg_tok - dt0), todo);
        for (u32 sub = 0; sub < f.pack; ++sub)
          for (u32 i = 0; i < k; ++i) {
            const u64 dk = dof + seg + sub * f.d_seg_bytes +
                           static_cast<u64>(dt0 + i) * f.d_tok_stride + f.d_base;
            zero_run(sink, zero, dk, f.unit, f.s_page);
            zero_run(sink, zero, dk + f.d_half, f.unit, f.s_page);
          }
        spos += k;
        dpos += k;
        todo -= k;
      }
      return;
    }
    case FILL_ATTN_TAIL: {  // every unwritten slot up to the end of the allocated blocks; runs
      const u32 end = static_cast<u32>(dn) * f.d_blk_tok;
      if (total >= end) return;
      const u64 zero = static_cast<u64>(id_at(sid, sn, 0)) * f.s_page;
      for (u32 dpos = total; dpos < end;) {
        const u32 dbi = dpos / f.d_blk_tok;
        const u64 seg = static_cast<u64>((dpos % f.d_blk_tok) / f.d_seg_tok) * f.pack * f.d_seg_bytes;
        const u32 dti = dpos % f.d_seg_tok;
        const u32 k = std::min(f.d_seg_tok - dti, end - dpos);
        const u64 dof = static_cast<u64>(id_at(did, dn, dbi)) * f.d_page;
        for (u32 sub = 0; sub < f.pack; ++sub) {
          const u64 dk = dof + seg + sub * f.d_seg_bytes + static_cast<u64>(dti) * f.d_tok_stride;
          zero_run(sink, zero, dk, static_cast<u64>(k) * f.unit, f.s_page);
          zero_run(sink, zero, dk + f.d_half, static_cast<u64>(k) * f.unit, f.s_page);
        }
        dpos += k;
      }
      return;
    }
    case FILL_HND_LAST: {  // per head, the tail of the last destination page
      if (total == 0) return;
      const u32 filled = total % f.d_blk_tok;
      if (filled == 0) return;
      const u64 len = static_cast<u64>(f.d_blk_tok - filled) * f.unit;
      const u64 zero = static_cast<u64>(id_at(sid, sn, 0)) * f.s_page;
      const u64 dof = static_cast<u64>(id_at(did, dn, total / f.d_blk_tok)) * f.d_page;
      for (u32 h = 0; h < f.heads; ++h) {
        const u64 dk = dof + f.d_base + h * f.d_head_stride + static_cast<u64>(filled) * f.unit;
        zero_run(sink, zero, dk, len, f.s_page);
        zero_run(sink, zero, dk + f.d_half, len, f.s_page);
      }
      return;
    }
    case FILL_HND_TAIL: {
      const u32 end = static_cast<u32>(dn) * f.d_blk_tok;
      if (total >= end) return;
      const u64 zero = static_cast<u64>(id_at(sid, sn, 0)) * f.s_page;
      for (u32 dpos = total; dpos < end;) {
        const u32 dbi = dpos / f.d_blk_tok, dti = dpos % f.d_blk_tok;
        const u32 k = std::min(f.d_blk_tok - dti, end - dpos);
        const u64 dof = static_cast<u64>(id_at(did, dn, dbi)) * f.d_page;
        for (u32 h = 0; h < f.heads; ++h) {
          const u64 dk = dof + h * f.d_head_stride + static_cast<u64>(dti) * f.unit;
          zero_run(sink, zero, dk, static_cast<u64>(k) * f.unit, f.s_page);
          zero_run(sink, zero, dk + f.d_half, static_cast<u64>(k) * f.unit, f.s_page);
        }
        dpos += k;
      }
      return;
    }
  }
}

void run_mla(const MlaOp& m, const kvt_task& t, const Groups& sg, const Groups& dg, Sink& sink) {
  const u32 *sid, *did;
  u64 sn, dn;
  sg.get(m.group, sid, sn);
  dg.get(m.group, did, dn);
  const bool last = t.reach_last_token != 0;
  if (m.equal_tp) {
    // whole manager blocks; an incomplete block waits for the next chunk, the last chunk
    // sends every remaining allocated block
    const u64 first = t.seen_tokens / m.s_mgr_tok;
    const u64 end = last ? sn : static_cast<u32>(t.seen_tokens + t.new_tokens) / m.s_mgr_tok;
    const u64 len = static_cast<u64>(m.s_mgr_tok) * m.tok_bytes;
    for (u64 i = first; i < end; ++i)
      sink.put(static_cast<u64>(id_at(sid, sn, i)) * m.s_page,
               static_cast<u64>(id_at(did, dn, i)) * m.d_page, len);
    return;
  }
  u32 pos = t.seen_tokens, rem = t.new_tokens;
  while (rem > 0) {
    const u32 ti = pos % m.kernel_tok;
    const u32 k = std::min(m.kernel_tok - ti, rem);
    if (k == m.kernel_tok || last || ti + k == m.kernel_tok)
      sink.put(static_cast<u64>(id_at(sid, sn, pos / m.s_mgr_tok)) * m.s_page +
                   static_cast<u64>((pos % m.s_mgr_tok) / m.kernel_tok) * m.kernel_bytes,
               static_cast<u64>(id_at(did, dn, pos / m.d_mgr_tok)) * m.d_page +
                   static_cast<u64>((pos % m.d_mgr_tok) / m.kernel_tok) * m.kernel_bytes,
               m.kernel_bytes);
    pos += k;
    rem -= k;
  }
  if (!m.pad || !last) return;
  const u64 total = static_cast<u64>(t.seen_tokens) + t.new_tokens;
  const u64 room = dn * static_cast<u64>(m.d_mgr_tok);
  if (total >= room) return;
  const u64 zero = static_cast<u64>(id_at(sid, sn, 0)) * m.s_page;
  for (u64 dpos = total; dpos < room;) {
    const u64 tib = dpos % m.d_mgr_tok;
    const u64 k = std::min<u64>(m.d_mgr_tok - tib, room - dpos);
    zero_run(sink, zero,
             static_cast<u64>(id_at(did, dn, dpos / m.d_mgr_tok)) * m.d_page + tib * m.tok_bytes,
             k * m.tok_bytes, m.s_page);
    dpos += k;
  }
}

int interpret(const kvt_parser& p, const kvt_task& task, kvt_block_lists* lists,
              kvt_run_lists* runs) {
  const Groups sg{task.src_blocks, task.src_group_len, task.n_src_groups};
  const Groups dg{task.dst_blocks, task.dst_group_len, task.n_dst_groups};
  const bool last = task.reach_last_token != 0;
  if (p.deferred_error != KVT_OK) return fail(p.deferred_error, p.deferred_msg);
  const size_t n_lists = lists ? lists->tensors.size() : runs->tensors.size();
  for (const Op& op : p.ops) {
    if (op.only_last && !last) continue;
    if (op.bad_shape) throw RangeError("state shape metadata too short");
    u32 tensor = 0;
    if (op.kind == OP_WALK) tensor = op.walk.tensor;
    if (tensor >= n_lists) throw RangeError("tensor index beyond the parser's list count");
    Sink sink{lists ? &lists->tensors[tensor] : nullptr, p.caps[tensor],
              runs ? &runs->tensors[tensor] : nullptr};
    switch (op.kind) {
      case OP_WALK: run_walk(op.walk, task, sg, dg, sink); break;
      case OP_PAGES: run_pages(op.pages, task, sg, dg, sink); break;
      case OP_STATE: run_state(op.state, sg, dg, sink); break;
      case OP_GDN: run_gdn(op.gdn, sg, dg, sink); break;
      case OP_FILL: run_fill(op.fill, task, sg, dg, sink); break;
      case OP_MLA: run_mla(op.mla, task, sg, dg, sink); break;
    }
  }
  return KVT_OK;
}

}  // namespace
}  // namespace kvt

using namespace kvt;

extern "C" {

int kvt_parser_create(int parser_id, const kvt_worker_info* src, const kvt_worker_info* dst,
                      uint32_t valid_mask, uint32_t kvt_tp_size, uint32_t kvt_tp_rank,
                      const kvt_parse_opts* opts, kvt_parser** out) {
  return guarded([&]() -> int {
    if (!src || !dst || !out) return fail(KVT_ERR_INVALID, "kvt_parser_create: null argument");
    if (src->n_tensors > KVT_MAX_TENSORS || dst->n_tensors > KVT_MAX_TENSORS)
      return fail(KVT_ERR_INVALID, "kvt_parser_create: too many cache tensors");
    if (src->worker_tp_rank >= KVT_MAX_TP_SIZE)
      return fail(KVT_ERR_INVALID, "kvt_parser_create: worker_tp_rank beyond MAX_TP_SIZE");
    if (parser_id < 0 || parser_id >= KVT_PARSER_COUNT)
      return fail(KVT_ERR_UNSUPPORTED, "kvt_parser_create: unknown parser id");
    if (src->engine_tp_size == 0 || dst->engine_tp_size == 0)
      return fail(KVT_ERR_INVALID, "kvt_parser_create: engine_tp_size must be positive");
    if (src->n_conv_state_shape > KVT_MAX_SHAPE_DIMS || src->n_ssm_state_shape > KVT_MAX_SHAPE_DIMS ||
        src->n_ple_conv_state_shape > KVT_MAX_SHAPE_DIMS ||
        src->n_gdn_conv_channel_dims > KVT_MAX_CHANNEL_DIMS ||
        src->n_ple_conv_channel_dims > KVT_MAX_CHANNEL_DIMS)
      return fail(KVT_ERR_INVALID, "kvt_parser_create: shape metadata count beyond the array size");
    std::unique_ptr<kvt_parser> p(new kvt_parser());
    kvt_parse_opts o{0, 1};
    if (opts) o = *opts;
    build_parser(parser_id, *src, *dst, valid_mask, kvt_tp_size, kvt_tp_rank, o, p.get());
    *out = p.release();
    return KVT_OK;
  });
}

void kvt_parser_destroy(kvt_parser* p) { delete p; }

int kvt_block_lists_create(kvt_block_lists** out) {
  if (!out) return fail(KVT_ERR_INVALID, "kvt_block_lists_create: null argument");
  *out = new kvt_block_lists();
  return KVT_OK;
}
void kvt_block_lists_destroy(kvt_block_lists* l) { delete l; }
void kvt_block_lists_clear(kvt_block_lists* l) {
  if (l) l->tensors.clear();
}
uint32_t kvt_block_lists_num_tensors(const kvt_block_lists* l) {
  return l ? static_cast<uint32_t>(l->tensors.size()) : 0;
}
int kvt_block_lists_view(const kvt_block_lists* l, uint32_t tensor, const kvt_ipc_block** data,
                         uint64_t* n) {
  if (!l || !data || !n) return fail(KVT_ERR_INVALID, "kvt_block_lists_view: null argument");
  if (tensor >= l->tensors.size())
    return fail(KVT_ERR_OUT_OF_RANGE, "kvt_block_lists_view: tensor index out of range");
  *data = l->tensors[tensor].data();
  *n = l->tensors[tensor].size();
  return KVT_OK;
}

int kvt_block_lists_append(kvt_block_lists* l, uint32_t tensor, const kvt_ipc_block* blocks,
                           uint64_t n) {
  return guarded([&]() -> int {
    if (!l || (!blocks && n)) return fail(KVT_ERR_INVALID, "kvt_block_lists_append: null argument");
    if (tensor >= KVT_MAX_TENSORS)
      return fail(KVT_ERR_OUT_OF_RANGE, "kvt_block_lists_append: tensor index out of range");
    if (l->tensors.size() <= tensor) l->tensors.resize(tensor + 1);
    l->tensors[tensor].insert(l->tensors[tensor].end(), blocks, blocks + n);
    return KVT_OK;
  });
}

int kvt_parse_block(const kvt_parser* p, const kvt_task* task, kvt_block_lists* lists) {
  return guarded([&]() -> int {
    if (!p || !task || !lists) return fail(KVT_ERR_INVALID, "kvt_parse_block: null argument");
    if (p->silent) return KVT_OK;
    if (lists->tensors.size() != p->n_lists) lists->tensors.resize(p->n_lists);
    return interpret(*p, *task, lists, nullptr);
  });
}

int kvt_parse_block_runs(const kvt_parser* p, const kvt_task* task, kvt_run_lists* lists) {
  return guarded([&]() -> int {
    if (!p || !task || !lists) return fail(KVT_ERR_INVALID, "kvt_parse_block_runs: null argument");
    if (p->silent) return KVT_OK;
    if (lists->tensors.size() != p->n_lists) lists->tensors.resize(p->n_lists);
    return interpret(*p, *task, nullptr, lists);
  });
}

}  // extern "C"
