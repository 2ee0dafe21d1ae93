// Concurrency driver for the host-side entry points of the library (test
// infrastructure; built by tests/test_host_fuzz.py with g++ -fsanitize=thread
// together with the product's host sources). The header promises that a parser
// is immutable once created and may be used from any number of threads, and
// that kvt_last_error() is the calling thread's own: here eight threads share
// three parsers (FLASH P==D, FLASH TP2 -> TP1, DPSK with an indexer tensor),
// each parses its share of a task set into lists of its own, merges,
// compresses, frames and un-frames them, every fourth task is made to fail, and
// everything is compared with what one thread computed beforehand. Any data
// race aborts the process.
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <thread>
#include <vector>

#include "kvt_hip.h"

#define CHECK(c)                                                          \
  do {                                                                    \
    if (!(c)) {                                                           \
      std::fprintf(stderr, "CHECK failed: %s (line %d)\n", #c, __LINE__); \
      std::abort();                                                       \
    }                                                                     \
  } while (0)

namespace {

struct Geometry {
  int parser_id;
  kvt_worker_info src, dst;
  uint32_t valid, tp_size, tp_rank;
  uint32_t groups;
};

kvt_worker_info flash_side(uint32_t tp, uint32_t rank, uint32_t heads_total, uint32_t nblk) {
  kvt_worker_info w;
  std::memset(&w, 0, sizeof(w));
  w.engine_tp_size = tp;
  w.worker_tp_rank = rank;
  w.n_tensors = 1;
  w.layer_num_blocks = nblk;
  w.token_sizes[0] = 2ull * (heads_total / tp) * 128 * 2;
  w.block_sizes[0] = w.token_sizes[0] * 16;
  w.num_layers = 2;
  w.attn_kernel_blk_ntpb = 16;
  w.attn_pack_size = 1;
  w.num_kv_heads = static_cast<int32_t>(heads_total);
  return w;
}

std::vector<Geometry> geometries() {
  std::vector<Geometry> g;
  g.push_back(Geometry{KVT_PARSER_FLASH_PEQD, flash_side(1, 0, 8, 256), flash_side(1, 0, 8, 300), 1u, 1, 0, 1});
  g.push_back(Geometry{KVT_PARSER_FLASH_PGTD, flash_side(2, 1, 8, 256), flash_side(1, 0, 8, 300), 3u, 2, 1, 1});
  kvt_worker_info s, d;
  std::memset(&s, 0, sizeof(s));
  s.engine_tp_size = 1;
  s.n_tensors = 2;
  s.layer_num_blocks = 256;
  s.token_sizes[0] = 1152;
  s.token_sizes[1] = 132;
  s.block_sizes[0] = 1152 * 64;
  s.block_sizes[1] = 132 * 64;
  s.num_layers = 2;
  s.attn_kernel_blk_ntpb = 64;
  s.indexer_blk_ntpb = 64;
  s.attn_pack_size = 1;
  s.num_kv_heads = 1;
  d = s;
  d.layer_num_blocks = 300;
  g.push_back(Geometry{KVT_PARSER_DPSK_PEQD, s, d, 1u, 1, 0, 1});
  return g;
}

struct Task {
  uint32_t seen, fresh, last;
  std::vector<uint32_t> src_blocks, dst_blocks;
  bool broken;
};

std::vector<Task> make_tasks(const Geometry& g, std::mt19937_64& rng, int n) {
  const uint32_t ntpb = static_cast<uint32_t>(g.src.block_sizes[0] / g.src.token_sizes[0]);
  std::vector<Task> out;
  for (int i = 0; i < n; ++i) {
    Task t;
    t.seen = static_cast<uint32_t>(rng() % 200);
    t.fresh = 1 + static_cast<uint32_t>(rng() % 900);
    t.last = static_cast<uint32_t>(rng() % 2);
    const uint32_t nb = (t.seen + t.fresh + ntpb - 1) / ntpb;
    for (uint32_t k = 0; k < nb; ++k) {
      t.src_blocks.push_back(static_cast<uint32_t>(rng() % g.src.layer_num_blocks));
      t.dst_blocks.push_back(static_cast<uint32_t>(rng() % g.dst.layer_num_blocks));
    }
    t.broken = i % 4 == 3;
    if (t.broken) t.src_blocks.back() = g.src.layer_num_blocks + 7 + static_cast<uint32_t>(i);
    out.push_back(std::move(t));
  }
  return out;
}

// Everything one task produces, as bytes, so that two runs compare with ==.
struct Result {
  int rc = 0;
  std::string error;
  std::vector<uint8_t> bytes;
};

void put(std::vector<uint8_t>& out, const void* p, size_t n) {
  const uint8_t* b = static_cast<const uint8_t*>(p);
  out.insert(out.end(), b, b + n);
}

Result run_task(const kvt_parser* p, const Geometry& g, const Task& t) {
  Result r;
  uint32_t sl = static_cast<uint32_t>(t.src_blocks.size()), dl = static_cast<uint32_t>(t.dst_blocks.size());
  kvt_task task{};
  task.seen_tokens = t.seen;
  task.new_tokens = t.fresh;
  task.reach_last_token = t.last;
  task.n_src_groups = g.groups;
  task.n_dst_groups = g.groups;
  task.src_blocks = t.src_blocks.data();
  task.dst_blocks = t.dst_blocks.data();
  task.src_group_len = &sl;
  task.dst_group_len = &dl;
  kvt_block_lists *l = nullptr, *back = nullptr, *expanded = nullptr;
  kvt_run_lists *runs = nullptr, *folded = nullptr;
  CHECK(kvt_block_lists_create(&l) == KVT_OK && kvt_block_lists_create(&back) == KVT_OK &&
        kvt_block_lists_create(&expanded) == KVT_OK);
  CHECK(kvt_run_lists_create(&runs) == KVT_OK && kvt_run_lists_create(&folded) == KVT_OK);
  r.rc = kvt_parse_block(p, &task, l);
  if (r.rc != KVT_OK) {
    r.error = kvt_last_error();
    CHECK(kvt_parse_block_runs(p, &task, runs) == r.rc);
    CHECK(r.error == kvt_last_error());
  } else {
    CHECK(kvt_parse_block_runs(p, &task, runs) == KVT_OK);
    CHECK(kvt_run_lists_expand(runs, expanded) == KVT_OK);
    CHECK(kvt_run_lists_compress(l, folded) == KVT_OK);
    const uint32_t nt = kvt_block_lists_num_tensors(l);
    for (uint32_t k = 0; k < nt; ++k) {
      const kvt_ipc_block *a = nullptr, *b = nullptr;
      uint64_t na = 0, nb = 0;
      CHECK(kvt_block_lists_view(l, k, &a, &na) == KVT_OK);
      CHECK(kvt_block_lists_view(expanded, k, &b, &nb) == KVT_OK);
      CHECK(na == nb && (na == 0 || std::memcmp(a, b, na * sizeof(*a)) == 0));
      put(r.bytes, a, na * sizeof(*a));
      const kvt_run* f = nullptr;
      uint64_t nf = 0;
      CHECK(kvt_run_lists_view(folded, k, &f, &nf) == KVT_OK);
      put(r.bytes, f, nf * sizeof(*f));
    }
    if (g.parser_id != KVT_PARSER_FLASH_PGTD) CHECK(kvt_block_lists_merge(l) == KVT_OK);
    kvt_wire_layout lay, lay2;
    CHECK(kvt_wire_layout_of(KVT_WIRE_TCP, l, &lay) == KVT_OK);
    std::vector<uint8_t> frame(lay.total_bytes);
    CHECK(kvt_wire_write_frame(KVT_WIRE_TCP, frame.data(), frame.size(), 11, 3, l, &lay) == KVT_OK);
    uint64_t reqid = 0, layer = 0;
    CHECK(kvt_wire_parse_frame(KVT_WIRE_TCP, frame.data(), frame.size(), nt, &reqid, &layer, back, &lay2) == KVT_OK);
    CHECK(reqid == 11 && layer == 3);
    for (uint32_t k = 0; k < nt; ++k) {
      const kvt_ipc_block* a = nullptr;
      uint64_t na = 0;
      CHECK(kvt_block_lists_view(back, k, &a, &na) == KVT_OK);
      put(r.bytes, a, na * sizeof(*a));
    }
    put(r.bytes, &lay2.total_bytes, sizeof(lay2.total_bytes));
  }
  kvt_run_lists_destroy(folded);
  kvt_run_lists_destroy(runs);
  kvt_block_lists_destroy(expanded);
  kvt_block_lists_destroy(back);
  kvt_block_lists_destroy(l);
  return r;
}

}  // namespace

int main(int argc, char** argv) {
  const int per_geometry = argc > 1 ? std::atoi(argv[1]) : 200;
  std::mt19937_64 rng(argc > 2 ? std::strtoull(argv[2], nullptr, 10) : 4242);
  const std::vector<Geometry> geo = geometries();
  std::vector<kvt_parser*> parsers(geo.size(), nullptr);
  std::vector<std::vector<Task>> tasks(geo.size());
  std::vector<std::vector<Result>> want(geo.size());
  long ok = 0, failed = 0;
  for (size_t i = 0; i < geo.size(); ++i) {
    kvt_parse_opts o{0, 1};
    CHECK(kvt_parser_create(geo[i].parser_id, &geo[i].src, &geo[i].dst, geo[i].valid, geo[i].tp_size,
                            geo[i].tp_rank, &o, &parsers[i]) == KVT_OK);
    tasks[i] = make_tasks(geo[i], rng, per_geometry);
    for (const Task& t : tasks[i]) {
      want[i].push_back(run_task(parsers[i], geo[i], t));
      CHECK((want[i].back().rc != KVT_OK) == t.broken);
      (want[i].back().rc == KVT_OK ? ok : failed)++;
    }
  }
  CHECK(ok > 0 && failed > 0);

  const int n_threads = 8;
  std::atomic<long> compared{0};
  std::vector<std::thread> pool;
  for (int tid = 0; tid < n_threads; ++tid)
    pool.emplace_back([&, tid] {
      // every thread walks every geometry, from a different starting task, so that the
      // same parser is inside parse_block on several threads at once; every second thread
      // also builds and destroys parsers of its own while the shared ones are in use
      for (int round = 0; round < 2; ++round)
        for (size_t i = 0; i < geo.size(); ++i) {
          kvt_parser* mine = nullptr;
          if (tid % 2) {
            kvt_parse_opts o{0, 1};
            CHECK(kvt_parser_create(geo[i].parser_id, &geo[i].src, &geo[i].dst, geo[i].valid, geo[i].tp_size,
                                    geo[i].tp_rank, &o, &mine) == KVT_OK);
          }
          const size_t n = tasks[i].size();
          for (size_t k = 0; k < n; ++k) {
            const size_t j = (k + static_cast<size_t>(tid) * 37) % n;
            const Result got = run_task(mine && (k & 1) ? mine : parsers[i], geo[i], tasks[i][j]);
            CHECK(got.rc == want[i][j].rc);
            CHECK(got.error == want[i][j].error);   // this thread's message, not a neighbour's
            CHECK(got.bytes == want[i][j].bytes);
            compared.fetch_add(1, std::memory_order_relaxed);
          }
          kvt_parser_destroy(mine);
        }
    });
  for (std::thread& t : pool) t.join();
  for (kvt_parser* p : parsers) kvt_parser_destroy(p);
  CHECK(compared.load() == static_cast<long>(n_threads) * 2 * static_cast<long>(geo.size()) * per_geometry);
  std::printf("thread check ok: %ld results compared on %d threads (%ld good, %ld failing tasks)\n",
              compared.load(), n_threads, ok, failed);
  return 0;
}
