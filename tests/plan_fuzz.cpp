// Robustness and correctness driver for the copy-plan builder (test infrastructure; built
// by tests/test_host_fuzz.py with hipcc, the HOST side under
// -fsanitize=address,undefined, together with the product sources). Runs without a GPU:
// every plan is created with device = KVT_DEVICE_NONE, which keeps the two chunk tables on
// the host.
//
// For random run lists (nested strides, lengths with any remainder, planted overshoots) and
// random chunk sizes, through kvt_plan_create_runs, kvt_plan_create_runs_bf16_to_fp8,
// kvt_plan_create and kvt_plan_create_objects:
//   * a run that leaves the stated capacity must be refused, nothing else may be;
//   * the tables of an accepted plan are walked with the kernels' own addressing
//     (csrc/kvt_kernels.hip: slices of 4 KiB, 16-byte vectors, multiply-high quotients);
//     every byte a kernel would touch must lie inside the stated capacity and the packed
//     layer, and the byte-to-byte mapping must equal the one obtained by expanding the runs
//     to plain ranges and concatenating them (the definition of pack / unpack).
// The index of the object ring (kvt_object_ring_*, host-only rings) gets random batches of
// keys as well: entries carry the key they were handed out for, so that a stale mapping shows.
#include <algorithm>
#include <csignal>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include <unistd.h>

#include "kvt_device.h"
#include "kvt_hip.h"

using kvt::Chunk;
using kvt::StrideShape;
using kvt::StrideTable;

static std::mt19937_64 rng(2024);
static uint64_t rnd(uint64_t n) { return n ? rng() % n : 0; }
static char g_case[512];
static void on_alarm(int) {
  const char msg[] = "plan_fuzz: case exceeded 30 s: ";
  (void)!write(2, msg, sizeof(msg) - 1);
  (void)!write(2, g_case, std::strlen(g_case));
  (void)!write(2, "\n", 1);
  _exit(3);
}
#define CHECK(c)                                                                        \
  do {                                                                                  \
    if (!(c)) {                                                                         \
      std::fprintf(stderr, "CHECK failed: %s (line %d) case: %s\n", #c, __LINE__, g_case); \
      std::abort();                                                                     \
    }                                                                                   \
  } while (0)

static uint32_t umulhi(uint32_t a, uint32_t b) {
  return static_cast<uint32_t>((static_cast<uint64_t>(a) * b) >> 32);
}

// Byte mapping of one table: for every packed byte of tensor t, the cache byte a kernel
// pairs it with (convert: the first of the two source bytes). side 0 = pack, 1 = unpack.
static void walk(const Chunk* table, uint64_t n, uint32_t chunk_bytes, const StrideTable* shapes,
                 int side, bool convert, const std::vector<uint64_t>& cap,
                 const std::vector<uint64_t>& tensor_bytes,
                 std::vector<std::vector<uint64_t>>& map) {
  const uint64_t scale = convert ? 2 : 1;
  for (uint64_t k = 0; k < n; ++k) {
    const Chunk& c = table[k];
    CHECK(c.len > 0 && c.len <= chunk_bytes);
    CHECK(c.tensor < cap.size());
    CHECK(c.packed + c.len <= tensor_bytes[c.tensor]);
    std::vector<uint64_t>& m = map[c.tensor];
    if (c.shape == 0) {
      CHECK(c.cache + scale * c.len <= cap[c.tensor]);
      for (uint32_t j = 0; j < c.len; ++j) {
        CHECK(m[c.packed + j] == ~0ull);  // every packed byte is produced exactly once
        m[c.packed + j] = c.cache + scale * j;
      }
      continue;
    }
    CHECK(c.shape <= kvt::kMaxShapes);
    const StrideShape& s = shapes->shape[c.shape - 1];
    CHECK(s.vlen > 0 && s.n_inner > 0 && c.len % 16 == 0 && c.cache % 16 == 0 && c.packed % 16 == 0);
    for (uint32_t v = 0; v < c.len / 16; ++v) {
      const uint32_t rec = s.vlen == 1 ? v : umulhi(v, s.inv_vlen);
      CHECK(rec == v / s.vlen);  // the reciprocal is exact over the chunk
      const uint32_t col = v - rec * s.vlen;
      const uint32_t o = rec / s.n_inner, i = rec % s.n_inner;
      // the reciprocal the pipelined kernels divide by (a divisor of 1 has none: they add the dividend)
      CHECK(s.n_inner == 1 ? s.inv_inner == 0 : umulhi(rec, s.inv_inner) == o);
      const uint64_t at = c.cache + o * s.outer[side] + i * s.inner[side] + col * 16 * scale;
      CHECK(at % 16 == 0 && at + 16 * scale <= cap[c.tensor]);
      for (uint32_t j = 0; j < 16; ++j) {
        CHECK(m[c.packed + 16ull * v + j] == ~0ull);
        m[c.packed + 16ull * v + j] = at + scale * j;
      }
    }
    // the word-wise path of the same chunk (4-byte aligned blobs) uses a second reciprocal
    for (uint32_t w = 0; w < c.len / 4; w += 1 + static_cast<uint32_t>(rnd(7)))
      CHECK(umulhi(w, s.inv_wlen) == w / (4 * s.vlen));
  }
}

// one past the last byte the run touches on either side (the generated runs cannot overflow)
static void extents(const kvt_run& r, uint64_t src_scale, uint64_t* s_end, uint64_t* d_end) {
  uint64_t s = r.src_offset, d = r.dst_offset;
  for (int k = 0; k < 3; ++k) {
    s += static_cast<uint64_t>(r.n[k] - 1) * r.src_stride[k];
    d += static_cast<uint64_t>(r.n[k] - 1) * r.dst_stride[k];
  }
  *s_end = s + src_scale * r.length;
  *d_end = d + r.length;
}

static kvt_run random_run(bool convert) {
  kvt_run r{};
  static const uint64_t lens[] = {16, 32, 48, 128, 256, 512, 1024, 2048, 4080, 4096, 8192, 20000,
                                  1, 7, 100, 1000, 3333};
  r.length = lens[rnd(sizeof(lens) / sizeof(lens[0]))];
  const bool aligned = rnd(4) != 0;
  const uint64_t unit = aligned ? 16 : (convert ? 2 : 1);
  r.src_offset = rnd(1 << 12) * unit;
  r.dst_offset = rnd(1 << 12) * unit;
  const uint64_t src_len = r.length * (convert ? 2 : 1);
  uint64_t s_span = src_len, d_span = r.length;  // bytes covered by the levels below
  for (int k = 2; k >= 0; --k) {
    static const uint32_t counts[3][6] = {{1, 1, 1, 2, 3, 5}, {1, 1, 2, 8, 16, 33}, {1, 1, 1, 2, 2, 4}};
    r.n[k] = counts[k][rnd(6)];
    if (r.n[k] > 1) {
      // strides at least as large as what lies below (no overlap), sometimes exactly that
      r.src_stride[k] = s_span + (rnd(3) ? rnd(64) * unit : 0);
      r.dst_stride[k] = d_span + (rnd(3) ? rnd(64) * unit : 0);
      if (aligned) {
        r.src_stride[k] = (r.src_stride[k] + 15) / 16 * 16;
        r.dst_stride[k] = (r.dst_stride[k] + 15) / 16 * 16;
      } else if (convert) {
        r.src_stride[k] += r.src_stride[k] & 1;
      }
      s_span = r.src_stride[k] * r.n[k];
      d_span = r.dst_stride[k] * r.n[k];
    }
  }
  return r;
}

static void fuzz_run_plans(int iters) {
  long accepted = 0, refused = 0, strided = 0, bytes = 0;
  for (int it = 0; it < iters; ++it) {
    const bool convert = rnd(3) == 0;
    const uint32_t n_t = 1 + static_cast<uint32_t>(rnd(3));
    static const uint32_t chunks[] = {0, 0, 4096, 8192, 32768, 65536, 524288};
    const uint32_t chunk = chunks[rnd(7)];
    std::snprintf(g_case, sizeof(g_case), "run plan it=%d convert=%d tensors=%u chunk=%u", it,
                  convert, n_t, chunk);
    alarm(30);
    kvt_run_lists* lists = nullptr;
    CHECK(kvt_run_lists_create(&lists) == KVT_OK);
    std::vector<uint64_t> s_cap(n_t, 0), d_cap(n_t, 0);
    // destination ranges of different runs must not collide for the mapping check: give
    // every run its own window on both sides
    for (uint32_t t = 0; t < n_t; ++t) {
      const uint32_t n_runs = static_cast<uint32_t>(rnd(6));
      uint64_t s_base = 0, d_base = 0;
      for (uint32_t k = 0; k < n_runs; ++k) {
        kvt_run r = random_run(convert);
        r.src_offset += s_base;
        r.dst_offset += d_base;
        uint64_t s_end, d_end;
        extents(r, convert ? 2 : 1, &s_end, &d_end);
        s_base = (s_end + 255) / 256 * 256;
        d_base = (d_end + 255) / 256 * 256;
        s_cap[t] = std::max(s_cap[t], s_end);
        d_cap[t] = std::max(d_cap[t], d_end);
        CHECK(kvt_run_lists_append(lists, t, &r, 1) == KVT_OK);
      }
      if (n_runs == 0) {
        const kvt_run none{};
        CHECK(kvt_run_lists_append(lists, t, &none, 0) == KVT_OK);
      }
    }
    // sometimes shave one byte off a capacity that is actually reached: must be refused
    int shaved = -1;
    if (rnd(4) == 0) {
      const uint32_t t = static_cast<uint32_t>(rnd(n_t));
      std::vector<uint64_t>& cap = rnd(2) ? s_cap : d_cap;
      if (cap[t] > 0) {
        cap[t] -= 1;
        shaved = static_cast<int>(t);
      }
    }
    kvt_plan* plan = nullptr;
    const int rc = convert ? kvt_plan_create_runs_bf16_to_fp8(KVT_DEVICE_NONE, lists, s_cap.data(),
                                                              d_cap.data(), chunk, &plan)
                           : kvt_plan_create_runs(KVT_DEVICE_NONE, lists, s_cap.data(),
                                                  d_cap.data(), chunk, &plan);
    if (shaved >= 0) {
      CHECK(rc == KVT_ERR_OUT_OF_RANGE && plan == nullptr);
      ++refused;
      kvt_run_lists_destroy(lists);
      continue;
    }
    CHECK(rc == KVT_OK && plan != nullptr);
    ++accepted;
    strided += kvt_plan_num_strided_chunks(plan) != 0;
    // expected mapping: expand to plain ranges, concatenate
    kvt_block_lists* plain = nullptr;
    CHECK(kvt_block_lists_create(&plain) == KVT_OK);
    CHECK(kvt_run_lists_expand(lists, plain) == KVT_OK);
    const void* chunks_p = nullptr;
    const void* shapes_p = nullptr;
    uint64_t n_chunks = 0;
    uint32_t cb = 0;
    CHECK(kvt_plan_host_tables(plan, &chunks_p, &n_chunks, &cb, &shapes_p) == KVT_OK);
    const Chunk* table = static_cast<const Chunk*>(chunks_p);
    const StrideTable* shapes = static_cast<const StrideTable*>(shapes_p);
    std::vector<uint64_t> tb(n_t);
    std::vector<std::vector<uint64_t>> pack_map(n_t), unpack_map(n_t);
    uint64_t layer_end = 0;
    for (uint32_t t = 0; t < n_t; ++t) {
      tb[t] = kvt_plan_tensor_bytes(plan, t);
      pack_map[t].assign(tb[t], ~0ull);
      unpack_map[t].assign(tb[t], ~0ull);
      CHECK(kvt_plan_tensor_offset(plan, t) % 256 == 0 && kvt_plan_tensor_offset(plan, t) >= layer_end);
      layer_end = kvt_plan_tensor_offset(plan, t) + tb[t];
    }
    CHECK(kvt_plan_layer_bytes(plan) >= layer_end);
    walk(table, n_chunks, cb, shapes, 0, convert, s_cap, tb, pack_map);
    walk(table + n_chunks, n_chunks, cb, shapes, 1, false, d_cap, tb, unpack_map);
    for (uint32_t t = 0; t < n_t; ++t) {
      const kvt_ipc_block* d = nullptr;
      uint64_t n = 0;
      CHECK(kvt_block_lists_view(plain, t, &d, &n) == KVT_OK);
      uint64_t cursor = 0;
      for (uint64_t k = 0; k < n; ++k)
        for (uint64_t j = 0; j < d[k].length; ++j, ++cursor) {
          CHECK(cursor < tb[t]);
          CHECK(pack_map[t][cursor] == d[k].src_offset + (convert ? 2 : 1) * j);
          CHECK(unpack_map[t][cursor] == d[k].dst_offset + j);
        }
      CHECK(cursor == tb[t]);
      bytes += static_cast<long>(cursor);
    }
    // the unpack table's writes ascend within a tensor
    for (uint64_t k = 1; k < n_chunks; ++k) {
      const Chunk &a = table[n_chunks + k - 1], &b = table[n_chunks + k];
      CHECK(a.tensor < b.tensor || (a.tensor == b.tensor && a.cache <= b.cache));
    }
    kvt_block_lists_destroy(plain);
    kvt_plan_destroy(plan);
    kvt_run_lists_destroy(lists);
  }
  alarm(0);
  std::printf("run plans: %ld accepted (%ld with strided chunks), %ld refused, %ld bytes mapped\n",
              accepted, strided, refused, bytes);
  CHECK(accepted > iters / 2 && strided > iters / 10 && refused > iters / 20);
}

static void fuzz_range_plans(int iters) {
  long accepted = 0, objects = 0;
  for (int it = 0; it < iters; ++it) {
    std::snprintf(g_case, sizeof(g_case), "range plan it=%d", it);
    alarm(30);
    static const uint32_t chunks[] = {0, 4096, 16384, 524288};
    const uint32_t chunk = chunks[rnd(4)];
    const bool as_objects = rnd(3) == 0;
    const uint64_t object = 4096 * (1 + rnd(8));
    kvt_block_lists* lists = nullptr;
    CHECK(kvt_block_lists_create(&lists) == KVT_OK);
    std::vector<kvt_ipc_block> v;
    uint64_t s = rnd(100), d = rnd(100), total = 0;
    const uint32_t n = static_cast<uint32_t>(rnd(12));
    for (uint32_t k = 0; k < n; ++k) {
      const uint64_t len = as_objects ? object : 1 + rnd(70000);  // an object = whole ranges
      v.push_back(kvt_ipc_block{s, d, len});
      s += len + rnd(3) * rnd(5000);
      d += len + rnd(3) * rnd(5000);
      total += len;
    }
    CHECK(kvt_block_lists_append(lists, 0, v.data(), v.size()) == KVT_OK);
    uint64_t s_cap = s, d_cap = d;
    kvt_plan* plan = nullptr;
    const uint64_t stride = object * (1 + rnd(4));
    const int rc = as_objects ? kvt_plan_create_objects(KVT_DEVICE_NONE, lists, &s_cap, &d_cap,
                                                        object, stride, chunk, &plan)
                              : kvt_plan_create(KVT_DEVICE_NONE, lists, &s_cap, &d_cap, nullptr,
                                                chunk, &plan);
    CHECK(rc == KVT_OK && plan != nullptr);
    ++accepted;
    objects += as_objects;
    const void* chunks_p = nullptr;
    const void* shapes_p = nullptr;
    uint64_t n_chunks = 0;
    uint32_t cb = 0;
    CHECK(kvt_plan_host_tables(plan, &chunks_p, &n_chunks, &cb, &shapes_p) == KVT_OK);
    const Chunk* table = static_cast<const Chunk*>(chunks_p);
    std::vector<uint64_t> tb{kvt_plan_tensor_bytes(plan, 0)};
    std::vector<std::vector<uint64_t>> pm(1), um(1);
    pm[0].assign(tb[0], ~0ull);
    um[0].assign(tb[0], ~0ull);
    walk(table, n_chunks, cb, static_cast<const StrideTable*>(shapes_p), 0, false, {s_cap}, tb, pm);
    walk(table + n_chunks, n_chunks, cb, static_cast<const StrideTable*>(shapes_p), 1, false,
         {d_cap}, tb, um);
    // byte k of the concatenated ranges sits at k (plain) or spread object by object
    uint64_t cursor = 0;
    for (const kvt_ipc_block& b : v)
      for (uint64_t j = 0; j < b.length; ++j, ++cursor) {
        const uint64_t at = as_objects ? (cursor / object) * stride + cursor % object : cursor;
        CHECK(at < tb[0] && pm[0][at] == b.src_offset + j && um[0][at] == b.dst_offset + j);
      }
    CHECK(cursor == total);
    if (as_objects && total)
      CHECK(tb[0] == (total / object - 1) * stride + object);
    else
      CHECK(tb[0] == total);
    kvt_plan_destroy(plan);
    kvt_block_lists_destroy(lists);
  }
  alarm(0);
  std::printf("range plans: %ld accepted, %ld as store objects\n", accepted, objects);
}

// Runs whose counts and strides are garbage (a run is 88 bytes however many ranges it stands
// for): every entry point must answer within the watchdog's limit and without exhausting memory.
static void fuzz_hostile_runs(int iters) {
  long accepted = 0;
  for (int it = 0; it < iters; ++it) {
    std::snprintf(g_case, sizeof(g_case), "hostile run it=%d", it);
    alarm(30);
    kvt_run r{};
    r.length = rnd(3) ? 1 + rnd(1 << 16) : 1 + rnd(1ull << 40);
    r.src_offset = rnd(1 << 20);
    r.dst_offset = rnd(1 << 20);
    for (int k = 0; k < 3; ++k) {
      static const uint32_t counts[] = {1, 2, 1000, 1u << 20, 0x7FFFFFFFu, 0xFFFFFFFFu};
      r.n[k] = counts[rnd(6)];
      r.src_stride[k] = rnd(3) ? rnd(1 << 16) : 0;
      r.dst_stride[k] = rnd(3) ? rnd(1 << 16) : 0;
    }
    kvt_run_lists* lists = nullptr;
    CHECK(kvt_run_lists_create(&lists) == KVT_OK);
    CHECK(kvt_run_lists_append(lists, 0, &r, 1) == KVT_OK);
    const uint64_t s_cap = rnd(2) ? ~0ull >> rnd(40) : rnd(1ull << 34);
    const uint64_t d_cap = rnd(1ull << 26);     // what an accepted plan may have to enumerate
    kvt_plan* plan = nullptr;
    const int rc = rnd(2) ? kvt_plan_create_runs(KVT_DEVICE_NONE, lists, &s_cap, &d_cap, 0, &plan)
                          : kvt_plan_create_runs_bf16_to_fp8(KVT_DEVICE_NONE, lists, &s_cap, &d_cap,
                                                             0, &plan);
    CHECK((rc == KVT_OK) == (plan != nullptr));
    if (plan) {
      ++accepted;
      CHECK(kvt_plan_tensor_bytes(plan, 0) <= d_cap);
      kvt_plan_destroy(plan);
    }
    kvt_block_lists* plain = nullptr;
    CHECK(kvt_block_lists_create(&plain) == KVT_OK);
    uint64_t ranges = 0;
    CHECK(kvt_run_lists_totals(lists, 0, &ranges, nullptr) == KVT_OK);
    const int rc2 = ranges <= (1u << 22) ? kvt_run_lists_expand(lists, plain) : KVT_ERR_INVALID;
    CHECK(rc2 == KVT_OK || rc2 == KVT_ERR_INVALID);
    kvt_block_lists_destroy(plain);
    kvt_run_lists_destroy(lists);
  }
  alarm(0);
  std::printf("hostile runs: %ld of %d accepted\n", accepted, iters);
}

// The object ring's index on host-only rings: every entry carries the key it was given for
// (written through the entry pointer when the ring asks for the block), so a lookup that
// names a stale or foreign entry is seen at once; exact-size key buffers let the sanitizer
// see a read past the last key.
static void fuzz_object_rings(int iters) {
  long reserved = 0, refused = 0, hits = 0;
  for (int it = 0; it < iters; ++it) {
    std::snprintf(g_case, sizeof(g_case), "object ring it=%d", it);
    const uint32_t n_entries = 1 + static_cast<uint32_t>(rnd(9));
    const uint32_t key_bytes = 1 + static_cast<uint32_t>(rnd(3) ? rnd(16) : rnd(256));
    const uint64_t entry_bytes = key_bytes + rnd(40);
    kvt_object_ring* r = nullptr;
    CHECK(kvt_object_ring_create(KVT_DEVICE_NONE, entry_bytes, n_entries, key_bytes, &r) == KVT_OK);
    const uint32_t universe = 2 + static_cast<uint32_t>(rnd(3 * n_entries));
    auto key_of = [&](uint32_t id, uint8_t* out) {
      for (uint32_t b = 0; b < key_bytes; ++b) out[b] = static_cast<uint8_t>((id * 131u + b * 7u) ^ (b < 4 ? id >> (8 * b) : 0));
    };
    // distinct ids must give distinct keys: with one-byte keys keep the universe small
    const uint32_t ids = key_bytes == 1 ? std::min<uint32_t>(universe, 2) : universe;
    for (int step = 0; step < 40; ++step) {
      const uint32_t n = static_cast<uint32_t>(rnd(2 * n_entries + 2));
      std::vector<uint32_t> id(n);
      std::vector<uint8_t> keys(static_cast<size_t>(n) * key_bytes);
      for (uint32_t i = 0; i < n; ++i) {
        id[i] = static_cast<uint32_t>(rnd(ids));
        key_of(id[i], keys.data() + static_cast<size_t>(i) * key_bytes);
      }
      std::vector<uint32_t> entries(n);
      std::vector<uint8_t> flag(n);
      const int rc = kvt_object_ring_reserve(r, keys.data(), n, entries.data(), flag.data());
      if (rc != KVT_OK) {
        CHECK(rc == KVT_ERR_INVALID);
        ++refused;
      } else {
        ++reserved;
        std::vector<uint32_t> fresh;
        for (uint32_t i = 0; i < n; ++i) {
          CHECK(entries[i] < n_entries);
          uint8_t* e = static_cast<uint8_t*>(kvt_object_ring_entry(r, entries[i]));
          CHECK(e != nullptr);
          if (flag[i]) {
            std::memcpy(e, keys.data() + static_cast<size_t>(i) * key_bytes, key_bytes);
            if (rnd(4)) fresh.push_back(entries[i]);
          } else {
            // stored already, or asked for earlier in this very call: either way the entry
            // holds this key
            CHECK(std::memcmp(e, keys.data() + static_cast<size_t>(i) * key_bytes, key_bytes) == 0);
          }
          for (uint32_t j = 0; j < i; ++j)   // same key, same entry; different keys, different entries
            CHECK((id[i] == id[j]) == (entries[i] == entries[j]));
        }
        CHECK(kvt_object_ring_commit(r, fresh.data(), static_cast<uint32_t>(fresh.size())) == KVT_OK);
        // what was not written is given up half of the time (written entries are left alone),
        // otherwise it stays reserved and narrows the ring
        if (rnd(2)) CHECK(kvt_object_ring_release(r, entries.data(), n) == KVT_OK);
      }
      const uint32_t m = static_cast<uint32_t>(rnd(6));
      std::vector<uint8_t> probe(static_cast<size_t>(m) * key_bytes);
      for (uint32_t i = 0; i < m; ++i) key_of(static_cast<uint32_t>(rnd(ids)), probe.data() + static_cast<size_t>(i) * key_bytes);
      std::vector<uint32_t> pe(m);
      std::vector<uint8_t> found(m);
      CHECK(kvt_object_ring_lookup(r, probe.data(), m, pe.data(), found.data()) == KVT_OK);
      for (uint32_t i = 0; i < m; ++i)
        if (found[i]) {
          ++hits;
          CHECK(pe[i] < n_entries);
          CHECK(std::memcmp(kvt_object_ring_entry(r, pe[i]), probe.data() + static_cast<size_t>(i) * key_bytes, key_bytes) == 0);
        }
    }
    kvt_object_ring_destroy(r);
  }
  std::printf("object rings: %ld batches reserved, %ld refused, %ld lookups hit\n", reserved, refused, hits);
  CHECK(reserved > iters && refused > 0 && hits > iters);
}

int main(int argc, char** argv) {
  std::signal(SIGALRM, on_alarm);
  const int scale = argc > 1 ? std::atoi(argv[1]) : 1;
  if (argc > 2) rng.seed(std::strtoull(argv[2], nullptr, 10));
  fuzz_run_plans(400 * scale);
  fuzz_range_plans(200 * scale);
  fuzz_hostile_runs(300 * scale);
  fuzz_object_rings(150 * scale);
  std::printf("plan fuzz ok\n");
  return 0;
}
