// Robustness driver for the host-side entry points of the library (test
// infrastructure; built by tests/test_host_fuzz.py with
// g++ -fsanitize=address,undefined together with the product's host sources).
// Feeds well-formed, mutated and garbage inputs through the C ABI and checks
// invariants; any memory error or undefined behaviour aborts the process.
//
//   wire   frames round-trip; mutated / truncated frames never read outside
//          the buffer and, when accepted, describe blobs inside it
//   runs   expand(compress(x)) == x on random lists with planted progressions
//   merge  output ascending in src, byte total preserved, no zero lengths
//   parse  random (also nonsensical) geometries for all 25 parser ids:
//          kvt_parse_block and kvt_parse_block_runs agree (same code, same
//          ranges after expansion) and never crash
#include <cstdio>
#include <cstdlib>
#include <algorithm>
#include <cstring>
#include <random>
#include <vector>

#include "kvt_hip.h"

#include <csignal>
#include <unistd.h>

static std::mt19937_64 rng(12345);

// Watchdog: a case that runs for more than 20 s is a hang (a loop whose trip count comes
// straight from untrusted metadata); say which case it was.
static char g_case[4096];
static void on_alarm(int) {
  const char msg[] = "host_fuzz: case exceeded 20 s: ";
  (void)!write(2, msg, sizeof(msg) - 1);
  (void)!write(2, g_case, std::strlen(g_case));
  (void)!write(2, "\n", 1);
  _exit(3);
}
static uint64_t rnd(uint64_t n) { return n ? rng() % n : 0; }
#define CHECK(c)                                                        \
  do {                                                                  \
    if (!(c)) {                                                         \
      std::fprintf(stderr, "CHECK failed: %s (line %d)\n", #c, __LINE__); \
      std::abort();                                                     \
    }                                                                   \
  } while (0)

static std::vector<kvt_ipc_block> view(const kvt_block_lists* l, uint32_t t) {
  const kvt_ipc_block* d = nullptr;
  uint64_t n = 0;
  CHECK(kvt_block_lists_view(l, t, &d, &n) == KVT_OK);
  return std::vector<kvt_ipc_block>(d, d + n);
}

static bool same(const std::vector<kvt_ipc_block>& a, const std::vector<kvt_ipc_block>& b) {
  return a.size() == b.size() &&
         (a.empty() || std::memcmp(a.data(), b.data(), a.size() * sizeof(kvt_ipc_block)) == 0);
}

static void fuzz_wire(int iters) {
  for (int it = 0; it < iters; ++it) {
    const int fmt = static_cast<int>(rnd(2));
    const uint32_t nt = fmt == KVT_WIRE_TCP ? 1 + static_cast<uint32_t>(rnd(8)) : 1;
    kvt_block_lists* l = nullptr;
    CHECK(kvt_block_lists_create(&l) == KVT_OK);
    for (uint32_t t = 0; t < nt; ++t) {
      std::vector<kvt_ipc_block> v(rnd(20));
      for (auto& b : v) b = kvt_ipc_block{rnd(1ull << 40), rnd(1ull << 40), 1 + rnd(200)};
      CHECK(kvt_block_lists_append(l, t, v.data(), v.size()) == KVT_OK);
    }
    kvt_wire_layout lay;
    CHECK(kvt_wire_layout_of(fmt, l, &lay) == KVT_OK);
    // exact-size heap buffer: the sanitizer sees any access one byte past the frame
    std::vector<uint8_t> frame(lay.total_bytes);
    CHECK(kvt_wire_write_frame(fmt, frame.data(), frame.size(), it, it * 3, l, &lay) == KVT_OK);
    for (uint32_t t = 0; t < nt; ++t)
      for (uint64_t i = 0; i < lay.blob_bytes[t]; ++i) frame[lay.blob_offset[t] + i] = static_cast<uint8_t>(rng());
    kvt_block_lists* back = nullptr;
    CHECK(kvt_block_lists_create(&back) == KVT_OK);
    uint64_t reqid = 0, layer = 0;
    kvt_wire_layout lay2;
    CHECK(kvt_wire_parse_frame(fmt, frame.data(), frame.size(), nt, &reqid, &layer, back, &lay2) == KVT_OK);
    CHECK(reqid == static_cast<uint64_t>(it) && layer == static_cast<uint64_t>(it) * 3);
    CHECK(std::memcmp(&lay, &lay2, sizeof(lay)) == 0);
    for (uint32_t t = 0; t < nt; ++t) CHECK(same(view(l, t), view(back, t)));
    // mutations
    for (int m = 0; m < 40; ++m) {
      std::vector<uint8_t> f2(frame.begin(), frame.begin() + rnd(frame.size() + 1));
      const int flips = static_cast<int>(rnd(4));
      for (int k = 0; k < flips && !f2.empty(); ++k) {
        const size_t pos = rnd(f2.size());
        if (rnd(3) == 0) f2[pos] = 0xFF; else f2[pos] ^= static_cast<uint8_t>(1u << rnd(8));
      }
      if (rnd(4) == 0 && f2.size() >= 36)  // plant a huge count in one of the size fields
        for (int k = 0; k < 8; ++k) f2[12 + 8 * rnd(3) + k] = 0xFF;
      std::vector<uint8_t> exact(f2);   // fresh exact-size allocation
      kvt_wire_layout l3;
      const int rc = kvt_wire_parse_frame(fmt, exact.empty() ? reinterpret_cast<const void*>(&l3) : exact.data(),
                                          exact.size(), static_cast<uint32_t>(rnd(3)) ? nt : 0,
                                          &reqid, &layer, back, &l3);
      if (rc == KVT_OK) {
        CHECK(l3.total_bytes <= exact.size());
        for (uint32_t t = 0; t < l3.n_tensors; ++t) {
          CHECK(l3.blob_offset[t] <= exact.size() && l3.blob_bytes[t] <= exact.size() - l3.blob_offset[t]);
          uint64_t sum = 0;
          for (const auto& b : view(back, t)) sum += b.length;
          CHECK(sum == l3.blob_bytes[t]);
        }
      } else {
        CHECK(rc == KVT_ERR_INVALID);
      }
    }
    kvt_block_lists_destroy(back);
    kvt_block_lists_destroy(l);
  }
}

static void fuzz_runs_and_merge(int iters) {
  for (int it = 0; it < iters; ++it) {
    std::vector<kvt_ipc_block> v;
    const int groups = 1 + static_cast<int>(rnd(12));
    for (int g = 0; g < groups; ++g) {
      const uint64_t s0 = rnd(1ull << 30), d0 = rnd(1ull << 30), len = 1 + rnd(512);
      const uint64_t n0 = 1 + rnd(3), n1 = 1 + rnd(6), n2 = 1 + rnd(3);
      const uint64_t ss[3] = {rnd(1 << 20), rnd(1 << 12), rnd(1 << 10)};
      const uint64_t ds[3] = {rnd(1 << 20), rnd(1 << 12), rnd(1 << 10)};
      for (uint64_t a = 0; a < n0; ++a)
        for (uint64_t b = 0; b < n1; ++b)
          for (uint64_t c = 0; c < n2; ++c)
            v.push_back(kvt_ipc_block{s0 + a * ss[0] + b * ss[1] + c * ss[2],
                                      d0 + a * ds[0] + b * ds[1] + c * ds[2], len});
    }
    kvt_block_lists *l = nullptr, *e = nullptr;
    kvt_run_lists* r = nullptr;
    CHECK(kvt_block_lists_create(&l) == KVT_OK && kvt_block_lists_create(&e) == KVT_OK);
    CHECK(kvt_run_lists_create(&r) == KVT_OK);
    CHECK(kvt_block_lists_append(l, 0, v.data(), v.size()) == KVT_OK);
    CHECK(kvt_run_lists_compress(l, r) == KVT_OK);
    CHECK(kvt_run_lists_expand(r, e) == KVT_OK);
    CHECK(same(view(e, 0), v));
    uint64_t nr = 0, nb = 0, total = 0;
    CHECK(kvt_run_lists_totals(r, 0, &nr, &nb) == KVT_OK);
    for (const auto& b : v) total += b.length;
    CHECK(nr == v.size() && nb == total);
    // merge: adjacent pieces of one long range, shuffled, plus the random list
    std::vector<kvt_ipc_block> m(v);
    uint64_t s = rnd(1 << 20), d = rnd(1 << 20);
    for (int k = 0; k < 10; ++k) {
      const uint64_t len = 1 + rnd(100);
      m.insert(m.begin() + rnd(m.size() + 1), kvt_ipc_block{(1ull << 41) + s, (1ull << 41) + d, len});
      s += len;
      d += len;
    }
    uint64_t n_out = 0, stats[4];
    uint64_t before = 0;
    for (const auto& b : m) before += b.length;
    CHECK(kvt_merge_interval(m.data(), m.size(), &n_out, stats) == KVT_OK);
    CHECK(n_out <= m.size());
    uint64_t after = 0;
    for (uint64_t i = 0; i < n_out; ++i) {
      CHECK(m[i].length > 0);
      if (i) CHECK(m[i - 1].src_offset <= m[i].src_offset);
      after += m[i].length;
    }
    CHECK(after <= before);   // overlapping prefixes may be dropped, nothing is invented
    kvt_run_lists_destroy(r);
    kvt_block_lists_destroy(e);
    kvt_block_lists_destroy(l);
  }
}

static uint64_t weird(uint64_t sane_max) {
  switch (rnd(10)) {
    case 0: return 0;
    case 1: return ~0ull >> rnd(40);
    default: return 1 + rnd(sane_max);
  }
}

static void fill_info(kvt_worker_info* w) {
  std::memset(w, 0, sizeof(*w));
  static const uint32_t tps[] = {1, 2, 4, 8, 3, 0};
  w->engine_tp_size = tps[rnd(6)];
  w->worker_tp_rank = static_cast<uint32_t>(rnd(9));
  w->n_tensors = static_cast<uint32_t>(rnd(4));
  w->layer_num_blocks = static_cast<uint32_t>(weird(64));
  for (int i = 0; i < KVT_MAX_TENSORS; ++i) {
    const uint64_t tok = weird(4096);
    w->token_sizes[i] = tok;
    w->block_sizes[i] = rnd(8) ? tok * (1 + rnd(64)) : weird(1 << 20);
  }
  w->num_layers = static_cast<uint32_t>(rnd(4));
  w->attn_kernel_blk_ntpb = static_cast<uint32_t>(weird(64));
  w->indexer_blk_ntpb = static_cast<uint32_t>(rnd(3) ? 0 : weird(64));
  w->attn_pack_size = static_cast<uint32_t>(rnd(4) ? 1 : weird(4));
  w->num_kv_heads = static_cast<int32_t>(rnd(34)) - 1;
  w->num_gdn_layers = static_cast<uint32_t>(rnd(4));
  w->hybrid_indexer_token_size = static_cast<uint32_t>(rnd(3) ? 0 : weird(256));
  w->gdn_conv_elem_size = static_cast<uint32_t>(weird(4));
  w->gdn_ssm_elem_size = static_cast<uint32_t>(weird(4));
  w->n_conv_state_shape = static_cast<uint32_t>(rnd(KVT_MAX_SHAPE_DIMS + 1));
  w->n_ssm_state_shape = static_cast<uint32_t>(rnd(KVT_MAX_SHAPE_DIMS + 1));
  w->n_gdn_conv_channel_dims = static_cast<uint32_t>(rnd(4));
  for (int i = 0; i < KVT_MAX_SHAPE_DIMS; ++i) {
    w->conv_state_shape[i] = weird(32);
    w->ssm_state_shape[i] = weird(16);
    w->ple_conv_state_shape[i] = weird(16);
  }
  for (int i = 0; i < KVT_MAX_CHANNEL_DIMS; ++i) {
    w->gdn_conv_channel_dims[i] = weird(16);
    w->ple_conv_channel_dims[i] = weird(16);
  }
  w->num_ple_layers = static_cast<uint32_t>(rnd(3));
  w->ple_block_group = static_cast<uint32_t>(rnd(6));
  w->ple_conv_elem_size = static_cast<uint32_t>(weird(4));
  w->n_ple_conv_state_shape = static_cast<uint32_t>(rnd(KVT_MAX_SHAPE_DIMS + 1));
  w->n_ple_conv_channel_dims = static_cast<uint32_t>(rnd(4));
  w->kda_conv_dim_first = static_cast<uint32_t>(rnd(2));
  w->hybrid_attn_token_size = static_cast<uint32_t>(rnd(3) ? 0 : weird(4096));
  w->kda_page_stride = rnd(3) ? 0 : weird(1 << 20);
}

// A mostly plausible pair of peers (the shapes the parsers are written for),
// then a few fields corrupted.
static void fill_sane_pair(kvt_worker_info* s, kvt_worker_info* d) {
  std::memset(s, 0, sizeof(*s));
  const uint32_t ntpb = 1u << rnd(7);
  const uint32_t heads_total = 1u << rnd(5);
  const uint32_t row = 16u << rnd(4);
  const uint32_t p_tp = 1u << rnd(4), d_tp = 1u << rnd(4);
  auto side = [&](kvt_worker_info* w, uint32_t tp) {
    std::memset(w, 0, sizeof(*w));
    w->engine_tp_size = tp;
    w->worker_tp_rank = static_cast<uint32_t>(rnd(tp));
    w->n_tensors = 1 + static_cast<uint32_t>(rnd(2));
    w->layer_num_blocks = 64 + static_cast<uint32_t>(rnd(64));
    const uint32_t heads = heads_total >= tp ? heads_total / tp : 1;
    w->token_sizes[0] = 2ull * heads * row;
    w->token_sizes[1] = 128;
    w->block_sizes[0] = w->token_sizes[0] * ntpb;
    w->block_sizes[1] = w->token_sizes[1] * ntpb;
    w->num_layers = 2;
    w->attn_pack_size = rnd(3) ? 1 : 2;
    w->attn_kernel_blk_ntpb = rnd(2) ? ntpb / w->attn_pack_size : std::max(1u, ntpb / 4);
    if (w->attn_kernel_blk_ntpb == 0) w->attn_kernel_blk_ntpb = 1;
    w->indexer_blk_ntpb = rnd(3) ? 0 : ntpb;
    w->num_kv_heads = static_cast<int32_t>(heads_total);
    w->num_gdn_layers = static_cast<uint32_t>(rnd(3));
    w->hybrid_indexer_token_size = 64;
    w->gdn_conv_elem_size = 2;
    w->gdn_ssm_elem_size = 4;
    w->n_conv_state_shape = 3;
    w->conv_state_shape[0] = 1; w->conv_state_shape[1] = 3; w->conv_state_shape[2] = 96 / tp * tp;
    w->n_ssm_state_shape = 4;
    w->ssm_state_shape[0] = 1; w->ssm_state_shape[1] = 4; w->ssm_state_shape[2] = 8; w->ssm_state_shape[3] = 8;
    w->n_gdn_conv_channel_dims = 3;
    w->gdn_conv_channel_dims[0] = w->gdn_conv_channel_dims[1] = w->gdn_conv_channel_dims[2] = 32;
    w->num_ple_layers = static_cast<uint32_t>(rnd(2));
    w->ple_block_group = w->num_gdn_layers + 2;
    w->ple_conv_elem_size = 2;
    w->n_ple_conv_state_shape = 3;
    w->ple_conv_state_shape[0] = 1; w->ple_conv_state_shape[1] = 2; w->ple_conv_state_shape[2] = 16;
    w->hybrid_attn_token_size = 576;
    w->kda_conv_dim_first = static_cast<uint32_t>(rnd(2));
  };
  side(s, p_tp);
  side(d, d_tp);
  d->num_gdn_layers = s->num_gdn_layers;
  d->num_ple_layers = s->num_ple_layers;
  d->ple_block_group = s->ple_block_group;
  for (int k = static_cast<int>(rnd(3)); k > 0; --k) {   // corrupt a few fields
    kvt_worker_info* w = rnd(2) ? s : d;
    switch (rnd(10)) {
      case 0: w->token_sizes[0] = weird(4096); break;
      case 1: w->block_sizes[0] = weird(1 << 20); break;
      case 2: w->attn_kernel_blk_ntpb = static_cast<uint32_t>(weird(64)); break;
      case 3: w->attn_pack_size = static_cast<uint32_t>(weird(5)); break;
      case 4: w->num_kv_heads = static_cast<int32_t>(rnd(40)) - 2; break;
      case 5: w->layer_num_blocks = static_cast<uint32_t>(weird(64)); break;
      case 6: w->n_tensors = static_cast<uint32_t>(rnd(4)); break;
      case 7: w->indexer_blk_ntpb = static_cast<uint32_t>(weird(64)); break;
      case 8: w->n_conv_state_shape = static_cast<uint32_t>(rnd(5)); break;
      default: w->conv_state_shape[2] = weird(64); break;
    }
  }
}

static void fuzz_parse(int iters) {
  long created = 0, parsed_ok = 0, ranges = 0;
  for (int it = 0; it < iters; ++it) {
    kvt_worker_info s, d;
    const bool sane = rnd(4) != 0;
    if (sane) {
      fill_sane_pair(&s, &d);
    } else {
      fill_info(&s);
      fill_info(&d);
    }
    const int pid = static_cast<int>(rnd(KVT_PARSER_COUNT + (sane ? 0 : 1)));
    kvt_parse_opts o{static_cast<uint32_t>(rnd(2)), static_cast<uint32_t>(rnd(2))};
    kvt_parser* p = nullptr;
    const uint32_t valid = sane && rnd(4) ? (s.engine_tp_size >= 32 ? ~0u : (1u << s.engine_tp_size) - 1u)
                                          : static_cast<uint32_t>(rng());
    const uint32_t tps = sane && rnd(4) ? s.engine_tp_size : static_cast<uint32_t>(rnd(9));
    const uint32_t tpr = sane && rnd(4) ? s.worker_tp_rank : static_cast<uint32_t>(rnd(9));
    const int rc = kvt_parser_create(pid, &s, &d, valid, tps, tpr, &o, &p);
    if (rc != KVT_OK) {
      CHECK(p == nullptr);
      continue;
    }
    ++created;
    for (int q = 0; q < 3; ++q) {
      const uint32_t want_groups = s.num_gdn_layers + 1 + (s.indexer_blk_ntpb ? 1 : 0) + s.num_ple_layers;
      const uint32_t ng_s = sane && rnd(5) ? want_groups : static_cast<uint32_t>(rnd(7));
      const uint32_t ng_d = rnd(5) ? ng_s : static_cast<uint32_t>(rnd(7));
      std::vector<uint32_t> sl(ng_s), dl(ng_d), sb, db;
      for (auto& x : sl) { x = static_cast<uint32_t>(rnd(40)); for (uint32_t k = 0; k < x; ++k) sb.push_back(static_cast<uint32_t>(rnd(8) ? rnd(64) : rng())); }
      for (auto& x : dl) { x = static_cast<uint32_t>(rnd(40)); for (uint32_t k = 0; k < x; ++k) db.push_back(static_cast<uint32_t>(rnd(8) ? rnd(64) : rng())); }
      kvt_task t{};
      t.seen_tokens = static_cast<uint32_t>(rnd(300));
      t.new_tokens = static_cast<uint32_t>(rnd(rnd(2) ? 40 : 600));
      t.reach_last_token = static_cast<uint32_t>(rnd(2));
      t.n_src_groups = ng_s;
      t.n_dst_groups = ng_d;
      // exact-size copies so that an index past the end is caught
      std::vector<uint32_t> sb2(sb), db2(db), sl2(sl), dl2(dl);
      t.src_blocks = sb2.data();
      t.dst_blocks = db2.data();
      t.src_group_len = sl2.data();
      t.dst_group_len = dl2.data();
      kvt_block_lists *l = nullptr, *e = nullptr;
      kvt_run_lists* r = nullptr;
      CHECK(kvt_block_lists_create(&l) == KVT_OK && kvt_block_lists_create(&e) == KVT_OK);
      CHECK(kvt_run_lists_create(&r) == KVT_OK);
      std::snprintf(g_case, sizeof(g_case),
                    "parser %d seen %u new %u last %u groups %u/%u  src: tp %u rank %u nt %u nblk %u B0 %llu T0 %llu "
                    "kb %u idx %u pack %u heads %d gdn %u ple %u attn_tok %u stride %llu | dst: tp %u rank %u nt %u nblk %u "
                    "B0 %llu T0 %llu kb %u idx %u pack %u",
                    pid, t.seen_tokens, t.new_tokens, t.reach_last_token, ng_s, ng_d, s.engine_tp_size,
                    s.worker_tp_rank, s.n_tensors, s.layer_num_blocks, (unsigned long long)s.block_sizes[0],
                    (unsigned long long)s.token_sizes[0], s.attn_kernel_blk_ntpb, s.indexer_blk_ntpb,
                    s.attn_pack_size, s.num_kv_heads, s.num_gdn_layers, s.num_ple_layers,
                    s.hybrid_attn_token_size, (unsigned long long)s.kda_page_stride, d.engine_tp_size,
                    d.worker_tp_rank, d.n_tensors, d.layer_num_blocks, (unsigned long long)d.block_sizes[0],
                    (unsigned long long)d.token_sizes[0], d.attn_kernel_blk_ntpb, d.indexer_blk_ntpb,
                    d.attn_pack_size);
      alarm(20);
      const int a = kvt_parse_block(p, &t, l);
      const int b = kvt_parse_block_runs(p, &t, r);
      alarm(0);
      CHECK(a == b);
      if (a == KVT_OK) {
        ++parsed_ok;
        CHECK(kvt_run_lists_expand(r, e) == KVT_OK);
        const uint32_t nt = kvt_block_lists_num_tensors(l);
        CHECK(nt == kvt_run_lists_num_tensors(r));
        for (uint32_t k = 0; k < nt; ++k) {
          CHECK(same(view(l, k), view(e, k)));
          ranges += static_cast<long>(view(l, k).size());
        }
      } else {
        CHECK(a == KVT_ERR_OUT_OF_RANGE || a == KVT_ERR_OVERFLOW || a == KVT_ERR_INVALID);
        CHECK(kvt_last_error()[0] != 0);
      }
      kvt_run_lists_destroy(r);
      kvt_block_lists_destroy(e);
      kvt_block_lists_destroy(l);
    }
    kvt_parser_destroy(p);
  }
  std::printf("parse: %ld parsers created, %ld tasks parsed, %ld ranges\n", created, parsed_ok, ranges);
  CHECK(created > iters / 50 && parsed_ok > iters / 50 && ranges > iters);
}

int main(int argc, char** argv) {
  std::signal(SIGALRM, on_alarm);
  const int scale = argc > 1 ? std::atoi(argv[1]) : 1;
  if (argc > 2) rng.seed(std::strtoull(argv[2], nullptr, 10));
  fuzz_wire(150 * scale);
  std::printf("wire ok\n");
  fuzz_runs_and_merge(300 * scale);
  std::printf("runs/merge ok\n");
  fuzz_parse(6000 * scale);
  std::printf("host fuzz ok\n");
  return 0;
}
