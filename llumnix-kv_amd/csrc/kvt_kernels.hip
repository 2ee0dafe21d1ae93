// Device kernels of libkvt_hip (gfx950 / CDNA4) and their launchers.
//
// Everything here is pure data movement and HBM-bound. The shape that measured
// fastest on MI355X, and that every kernel below follows:
//   * one workgroup = 256 lanes (4 wavefronts of 64) moves ONE 4 KiB slice:
//     a single 16-byte non-temporal load and store per lane, no loop. Many
//     short workgroups keep far more independent requests in flight than a few
//     long ones, and neighbouring slices reach DRAM close together in time;
//   * work is ordered by ascending cache address (the plan builder sorts), so
//     scattered reads / writes still walk DRAM pages in order;
//   * workgroup ids are dealt round-robin to the 8 XCDs, so id b is remapped to
//     (b % 8) * ceil(n / 8) + b / 8: each XCD then streams through one
//     contiguous eighth of the work list instead of touching every page.
// A launch limited to a share of the device runs instead as a few persistent workgroups (at
// best one per CU) that pipeline whole table entries over three register sets (an entry per
// workgroup, or per wavefront where entries are 4 or 8 KiB) and take them
// in order from one counter per XCD: what keeps such a launch fast is that the addresses in
// flight stay in one narrow window, as the order of dispatch keeps them in the unlimited shape.
// No MFMA, and LDS only to hand a ticket to the wavefronts of a workgroup: the HND<->NHD
// transform moves whole 16-byte vectors of rows that are contiguous on both sides, so it is
// a pure index permutation.
#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "kvt_device.h"

namespace kvt {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kThreads = 256;
constexpr uint32_t kSlice = kThreads * 16;  // bytes moved by one workgroup
constexpr uint32_t kSliceShift = 12;

__device__ __forceinline__ uint32_t xcd_remap(uint32_t b, uint32_t n) {
  const uint32_t per = (n + 7u) >> 3;
  return (b & 7u) * per + (b >> 3);
}

// Every pointer a kernel here follows is device-visible global memory, also where the
// compiler cannot tell (layer pointers are loaded from a table): saying so gives global
// instead of generic ("flat") memory instructions.
typedef __attribute__((address_space(1))) u32x4 g_u32x4;
__device__ __forceinline__ u32x4 load_vec(const uint8_t* p) {
  return __builtin_nontemporal_load((const g_u32x4*)(p));
}
// Plain instead of non-temporal loads, for a caller that reads the same data more than once
// within the reach of the 256 MiB memory-side cache (one layer sent to several destinations,
// stored and sent): a plain load leaves its line in the cache for the next reader, a
// non-temporal one does not. Measured on MI355X, one request of n tokens packed over 32
// layers, non-temporal against plain loads, microseconds per launch:
//   data not cached (cycling over 1-4 GiB):     32 MiB 16.0 / 16.1, 64 MiB 26.2 / 27.0,
//                                               128 MiB 50.9 / 53.4, 256 MiB 92.1 / 97.7
//   right after a kernel wrote the blocks:      32 MiB 12.9 / 13.2, 64 MiB 21.9 / 22.5,
//                                               128 MiB 44.0 / 46.6, 256 MiB 80.8 / 99.1
//   the same request again (back to back):      64 MiB 21.4 / 19.1, 128 MiB 45.4 / 42.5,
//                                               256 MiB 84.0 / 77.5, 512 MiB 163 / 171
// Non-temporal loads are the default: they win whenever the data is read once, also when a
// producer's stores have just left it in the cache. The launcher switches by the launch's
// payload against a limit the caller sets (kvt_set_copy_cached_load_max, 0 by default).
__device__ __forceinline__ u32x4 load_vec_temporal(const uint8_t* p) { return *(const g_u32x4*)(p); }
// Stores are non-temporal and written through at system scope (sc0 sc1 nt): nothing of a
// streamed copy is worth keeping in a cache. There is no builtin for that combination on a
// global store. Measured on MI355X against the compiler's non-temporal store (nt alone):
// config 2 pack 6.72 -> 6.87 TB/s, unpack 6.04 -> 6.10; config 1's unpack 24.2 -> 22.5 us.
__device__ __forceinline__ void store_vec(uint8_t* p, u32x4 v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1 nt" ::"v"(p), "v"(v) : "memory");
}

// Copies len (<= 4096) bytes with the whole workgroup when the two sides are not both
// 16-byte aligned: 4-byte words where possible, else bytes.
__device__ __forceinline__ void copy_slice_odd(uint8_t* __restrict__ dst,
                                               const uint8_t* __restrict__ src, uint32_t len,
                                               uint32_t tid) {
  const uintptr_t mis = reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src);
  if ((mis & 3u) == 0) {
    const uint32_t nw = len >> 2;
    const uint32_t* __restrict__ s = reinterpret_cast<const uint32_t*>(src);
    uint32_t* __restrict__ d = reinterpret_cast<uint32_t*>(dst);
#pragma clang loop vectorize(disable) unroll(disable)
    for (uint32_t i = tid; i < nw; i += kThreads) d[i] = s[i];
    const uint32_t done = nw << 2;
    if (tid < len - done) dst[done + tid] = src[done + tid];
  } else {
#pragma clang loop vectorize(disable) unroll(disable)
    for (uint32_t j = tid; j < len; j += kThreads) dst[j] = src[j];
  }
}

// Copies len (<= 4096) bytes with the whole workgroup. Fast path: 16-byte
// aligned on both sides; one vector per lane, stragglers byte-wise.
__device__ __forceinline__ void copy_slice(uint8_t* __restrict__ dst,
                                           const uint8_t* __restrict__ src, uint32_t len,
                                           uint32_t tid) {
  const uintptr_t mis = reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src);
  if ((mis & 15u) != 0) return copy_slice_odd(dst, src, len, tid);
  const uint32_t nvec = len >> 4;
  if (tid < nvec) store_vec(dst + (tid << 4), load_vec(src + (tid << 4)));
  const uint32_t done = nvec << 4;
  if (tid < len - done) dst[done + tid] = src[done + tid];
}

// ------------------------------------------------------------ chunk kernels
//
// Workgroup item b of a layer handles slice (b & mask) of table entry (b >> sub_shift);
// entries hold at most 4096 << sub_shift bytes, so a shorter one simply leaves its last
// workgroups idle. The normal launch has one workgroup per (slice, layer) item: grid (slices
// rounded up to 8, layers). A launch capped to a share of the device (CAPPED) has a
// one-dimensional grid of that many workgroups, a multiple of 8, which stride over the same
// items layer by layer; since the stride and the rounded slice count are both multiples of 8,
// a workgroup keeps meeting slices of the eighth that belongs to its XCD.
//
// A capped workgroup is persistent, and with one 16-byte vector per lane in flight its rate
// would follow the number of resident wavefronts (half the wave slots, half the rate), each
// item paying for three dependent loads in a row (table entry, layer pointer, data). So it
// takes kBatch items per trip in phases: the kBatch table entries (independent scalar
// loads), then the kBatch layer pointers, then the lanes' addresses, then the kBatch vector
// loads back to back; the stores of a trip are issued only after the loads of the next one
// (three register sets in rotation), so a lane has up to 2 x kBatch x 16 bytes in flight.

// This workgroup's way through the (item, layer) pairs of a launch: the items of a layer are
// dealt to the XCDs in eighths. Without tickets a workgroup strides through its XCD's pairs by
// the number of workgroups there. With tickets (eight counters, one per XCD, 128 bytes apart,
// zero at the start of the launch) it takes whatever pair is next on its XCD: workgroups that
// fall behind no longer spread the addresses in flight over a widening window, which is worth
// 16 % on a plain 4 GiB copy by 256 persistent workgroups (5.5 -> 6.4 TB/s). The last
// workgroup to leave zeroes the counters again (kTicketDone counts the leavers).
constexpr uint32_t kTicketStride = 32, kTicketDone = 8 * kTicketStride;  // in 32-bit words
// log2 of the 4 KiB slices one ticket stands for: 32 KiB. Finer tickets run into the rate at
// which one counter can be bumped (16 KiB entries, one per ticket: 11 % slower than without
// tickets), coarser ones give the order away again (64 / 128 KiB: -6 / -9 % on config 2).
constexpr uint32_t kTicketSlicesLog2 = 3;
struct EntryWalk {
  uint32_t n_items, n_layers, per8, xcd, step_layer, step_within, layer, within;
  uint32_t* tickets;
  uint32_t run_shift;  // a ticket stands for 1 << run_shift consecutive pairs
  uint32_t pair, left; // tickets: the next pair of the current run, and how many of it are left
  uint32_t turn;       // which LDS word carries the next ticket
  uint32_t ahead;      // lane 0: the ticket of the next run, asked for one run early
  // slices_log2: log2 of the 4 KiB slices one item holds
  __device__ __forceinline__ EntryWalk(uint32_t items, uint32_t layers, uint32_t* ticket_block, uint32_t slices_log2)
      : n_items(items), n_layers(layers), tickets(ticket_block), pair(0), left(0), turn(0), ahead(0) {
    per8 = (n_items + 7u) >> 3;
    xcd = blockIdx.x & 7u;
    run_shift = slices_log2 < kTicketSlicesLog2 ? kTicketSlicesLog2 - slices_log2 : 0u;
    if (tickets && threadIdx.x == 0) ahead = atomicAdd(tickets + xcd * kTicketStride, 1u);
    const uint32_t nloc = gridDim.x >> 3;  // workgroups per XCD
    step_layer = nloc / per8;
    step_within = nloc - step_layer * per8;
    layer = (blockIdx.x >> 3) / per8;
    within = (blockIdx.x >> 3) - layer * per8;
  }
  // The next pair, clamped to the last one past the end (`valid` false: nothing to move there);
  // returns false once the workgroup is past the last layer. A ticket travels from lane 0 to
  // the workgroup through one of two LDS words in turn: lane 0 cannot write a word again
  // before every wavefront has passed the barrier behind the other one, i.e. has read it.
  __device__ __forceinline__ bool next(uint32_t& item, uint32_t& lay, bool& valid) {
    if (tickets) {
      if (left == 0) {
        __shared__ uint32_t slot[2];
        if (threadIdx.x == 0) {
          slot[turn] = ahead;
          ahead = atomicAdd(tickets + xcd * kTicketStride, 1u);
        }
        __syncthreads();
        pair = __builtin_amdgcn_readfirstlane(slot[turn]) << run_shift;
        left = 1u << run_shift;
        turn ^= 1u;
      }
      layer = pair / per8;
      within = pair - layer * per8;
      ++pair;
      --left;
    }
    const bool live = layer < n_layers;
    const uint32_t b = xcd * per8 + within;
    valid = live && b < n_items;
    lay = min(layer, n_layers - 1u);
    item = min(b, n_items - 1u);
    if (!tickets) {
      within += step_within;
      layer += step_layer;
      const bool wrap = within >= per8;
      within -= wrap ? per8 : 0u;
      layer += wrap ? 1u : 0u;
    }
    return live;
  }
  // Call once, when next() has returned false.
  __device__ __forceinline__ void leave() {
    if (!tickets || threadIdx.x != 0) return;
    asm volatile("" ::"v"(ahead));  // the last ticket asked for has been handed out: it came back
    if (atomicAdd(tickets + kTicketDone, 1u) == gridDim.x - 1u) {
#pragma unroll
      for (uint32_t x = 0; x < 8; ++x) atomicExch(tickets + x * kTicketStride, 0u);
      atomicExch(tickets + kTicketDone, 0u);
    }
  }
};

// Three register sets in rotation: the loads of item k+1 are issued before the stores of item k,
// and a set is loaded again only two trips after its stores were issued.
// The compiler may reorder loads and stores that cannot alias, and it does: in some stages it
// issues a trip's stores in front of the loads that were to overlap them (it also sinks loads
// from a __restrict__ pointer behind the loop's exit test). FENCE pins the order as written;
// it needs the loads' base not to be a __restrict__ pointer. Measured, the pinned order gains
// 1-2 % on the plain tables (a changed kernel body had lost 5 % to a worse reordering) and
// loses 2 % on the strided ones at one workgroup per CU, which therefore stay as the compiler
// arranges them.
#define KVT_ISSUE_FENCE()              \
  do {                                 \
    asm volatile("" ::: "memory");     \
    __builtin_amdgcn_sched_barrier(0); \
  } while (0)
#define KVT_NO_FENCE() \
  do {                 \
  } while (0)
#define KVT_ROTATE3_WITH(NEXT, LOAD, STORE, FENCE) \
  do {                                             \
    if (!NEXT(0)) break;                           \
    LOAD(0);                                       \
    for (;;) {                                     \
      const bool l1 = NEXT(1);                     \
      LOAD(1);                                     \
      FENCE();                                     \
      STORE(0);                                    \
      FENCE();                                     \
      if (!l1) break;                              \
      const bool l2 = NEXT(2);                     \
      LOAD(2);                                     \
      FENCE();                                     \
      STORE(1);                                    \
      FENCE();                                     \
      if (!l2) break;                              \
      const bool l0 = NEXT(0);                     \
      LOAD(0);                                     \
      FENCE();                                     \
      STORE(2);                                    \
      FENCE();                                     \
      if (!l0) break;                              \
    }                                              \
  } while (0)
#define KVT_ROTATE3(NEXT, LOAD, STORE) KVT_ROTATE3_WITH(NEXT, LOAD, STORE, KVT_NO_FENCE)
#define KVT_ROTATE3_PINNED(NEXT, LOAD, STORE) KVT_ROTATE3_WITH(NEXT, LOAD, STORE, KVT_ISSUE_FENCE)

constexpr int kBatch = 4;
// How a chunk kernel walks its items: one workgroup per (slice, layer); a capped grid striding
// over them kBatch at a time; the same with the trips software-pipelined. Twice the bytes in
// flight pay below half the device (config 4 at a quarter: 4.8 / 4.5 -> 5.2 / 5.2 TB/s) and
// cost from there on (at one half 5.6 / 5.5 -> 5.1 / 5.2), so the launcher picks by grid size.
enum { kOnePerSlice = 0, kStriding = 1, kPipelined = 2 };
// in a kernel's sub_shift argument: Launch::temporal, Launch::cached_store (the launchers'
// `policy` argument, bits 0 and 1, shifted by 8)
constexpr uint32_t kTemporalFlag = 0x100u, kCachedStoreFlag = 0x200u;

// The uniform arguments of a chunk launch.
struct Launch {
  uint32_t n_slices, sub_shift;
  uint8_t* const* layer_ptrs;
  uint32_t n_tensors, first_layer, n_layers;
  uint8_t* packed;
  uint64_t layer_stride;
  const BlobOffsets* blobs;
  bool temporal;  // plain instead of non-temporal loads (bit 8 of the sub_shift argument)
  bool cached_store;  // plain stores, which leave their lines in the caches (bit 9)
  uint32_t* tickets;  // a capped launch: its block of counters, or nullptr (EntryWalk)
};

// A table entry as the kernels read it: the Chunk's two 16-bit fields as one word (a 16-bit
// field would be fetched with a vector load, everything else here with scalar loads).
struct __attribute__((may_alias, aligned(16))) Entry {
  uint64_t cache, packed;
  uint32_t len, tensor_t0, shape, reserved;
  __device__ __forceinline__ uint32_t tensor() const { return tensor_t0 & 0xFFFFu; }
  __device__ __forceinline__ uint32_t t0() const { return tensor_t0 >> 16; }
};
// Read as one 32-byte scalar load (field by field the compiler fetches the half it needs
// first and the rest a round trip later).
typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));
__device__ __forceinline__ u32x8 fetch_entry(const void* table, uint32_t e) {
  return static_cast<const u32x8*>(table)[e];
}
__device__ __forceinline__ Entry entry_of(u32x8 r) {
  Entry c;
  c.cache = r[0] | (static_cast<uint64_t>(r[1]) << 32);
  c.packed = r[2] | (static_cast<uint64_t>(r[3]) << 32);
  c.len = r[4];
  c.tensor_t0 = r[5];
  c.shape = r[6];
  c.reserved = r[7];
  return c;
}
static_assert(sizeof(Entry) == sizeof(Chunk) && offsetof(Chunk, tensor) == offsetof(Entry, tensor_t0) &&
                  offsetof(Chunk, t0) == offsetof(Entry, tensor_t0) + 2 &&
                  offsetof(Chunk, shape) == offsetof(Entry, shape),
              "Entry must mirror Chunk");

// One (slice, layer) item, uniform across the workgroup.
struct Item {
  Entry c;
  uint8_t* cache;  // the layer tensor's base + c.cache
  uint8_t* pk;     // where the entry's packed bytes start in this layer
  uint32_t sub;    // slice index inside the entry
};

// One lane's vector move: uniform base addresses (they stay in scalar registers) plus the
// lane's byte offsets. `on` = the lane has a vector to move.
struct Move {
  const uint8_t* src;
  uint8_t* dst;
  uint64_t src_off, dst_off;
  bool on;
};
#define KVT_NO_MOVE (Move{nullptr, nullptr, 0, 0, false})

// `fetch_table(entry)` reads a table entry; `place(item)` turns an item into the lane's move. Odd
// cases (misaligned slices, stragglers behind the last whole vector) `place` may move itself.
template <int MODE, class Fetch, class Place>
__device__ __forceinline__ void for_items(const Launch& L, Fetch fetch_table, Place place) {
  if (MODE == kOnePerSlice) {
    // A workgroup's life is a chain of dependent round trips and then its one vector, and
    // 2 048 resident workgroups have to hide all of it: the chain is kept to three links.
    // (1) every argument; (2) the table entry as ONE 32-byte scalar load and, beside it, the
    // layer pointer and blob position of tensor 0 (the only tensor of most plans: an entry of
    // another tensor pays one more link); (3) the data. There is no branch before the last
    // of these loads has been issued: a workgroup beyond the last slice (the grid is rounded
    // up to a multiple of 8) runs the same code on the last entry with a length of zero.
    // The empty asm statements pin where the loads complete: without them the compiler moves
    // a load next to its first use, behind the branch on the tensor index, and the chain grows
    // by a link.
    const uint32_t b = xcd_remap(blockIdx.x, L.n_slices), layer = blockIdx.y;
    const uint32_t bc = min(b, L.n_slices - 1u);
    uint64_t stride = L.layer_stride, blob = L.blobs->off[0];
    asm volatile("" : "+s"(stride), "+s"(blob));
    uint8_t* const* row = L.layer_ptrs + static_cast<uint64_t>(L.first_layer + layer) * L.n_tensors;
    u32x8 raw = fetch_table(bc >> L.sub_shift);
    uint8_t* base = row[0];
    asm volatile("" : "+s"(raw), "+s"(base));
    Item it;
    it.c = entry_of(raw);
    it.sub = bc & ((1u << L.sub_shift) - 1u);
    const uint32_t t = it.c.tensor();
    if (__builtin_expect(t != 0u, 0)) {
      base = row[t];
      blob = L.blobs->off[t];
    }
    it.cache = base + it.c.cache;
    it.pk = L.packed + layer * stride + blob + it.c.packed;
    if (b >= L.n_slices) it.c.len = 0;
    const Move m = place(it);
    if (m.on) {
      const uint8_t* src = m.src + m.src_off;
      u32x4 v;
      if (L.temporal) {
        v = load_vec_temporal(src);
      } else {
        // Written out: given the builtin, the compiler merges the two arms into ONE load and
        // drops the non-temporal hint with it.
        asm volatile("global_load_dwordx4 %0, %1, off nt\n\ts_waitcnt vmcnt(0)"
                     : "=v"(v)
                     : "v"(src)
                     : "memory");
      }
      if (L.cached_store)
        *(g_u32x4*)(m.dst + m.dst_off) = v;
      else
        store_vec(m.dst + m.dst_off, v);
    }
    return;
  }
  // lanes without a vector load from here: the layer pointer table, at least 16 bytes long
  const uint8_t* const idle = reinterpret_cast<const uint8_t*>(L.layer_ptrs);
  // the (slice, layer) pairs of this workgroup, one 4 KiB slice each: strided by the grid, or
  // in runs of eight neighbouring slices by ticket
  EntryWalk walk(L.n_slices, L.n_layers, L.tickets, 0);
  // kStriding: a trip loads kBatch vectors and stores them. kPipelined: three sets of kBatch
  // vectors in rotation (KVT_ROTATE3), the loads of the next kBatch items in flight before the
  // stores of the last ones are issued. What a set keeps until its stores is each vector's
  // destination (null: no vector).
  uint8_t* dst[3][kBatch];
  u32x4 r[3][kBatch];
  auto fetch = [&](int k) -> bool {
    bool live = false;
    Item it[kBatch];
    uint32_t lay[kBatch];
    bool valid[kBatch];
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {  // which items, and their table entries
      uint32_t bc;
      const bool more = walk.next(bc, lay[j], valid[j]);
      if (j == 0) live = more;
      it[j].c = entry_of(fetch_table(bc >> L.sub_shift));
      it[j].sub = bc & ((1u << L.sub_shift) - 1u);
    }
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {  // their layer tensors
      it[j].cache =
          L.layer_ptrs[static_cast<uint64_t>(L.first_layer + lay[j]) * L.n_tensors + it[j].c.tensor()] +
          it[j].c.cache;
      it[j].pk = L.packed + lay[j] * L.layer_stride + L.blobs->off[it[j].c.tensor()] + it[j].c.packed;
    }
    Move m[kBatch];
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      m[j] = KVT_NO_MOVE;
      if (valid[j]) m[j] = place(it[j]);
    }
#pragma unroll
    for (int j = 0; j < kBatch; ++j) r[k][j] = load_vec(m[j].on ? m[j].src + m[j].src_off : idle);
#pragma unroll
    for (int j = 0; j < kBatch; ++j) dst[k][j] = m[j].on ? m[j].dst + m[j].dst_off : nullptr;
    return live;
  };
  auto nothing = [](int) {};
  auto store = [&](int k) {
#pragma unroll
    for (int j = 0; j < kBatch; ++j)
      if (dst[k][j]) store_vec(dst[k][j], r[k][j]);
  };
  if (MODE == kStriding) {
    while (fetch(0)) store(0);
  } else {
    KVT_ROTATE3(fetch, nothing, store);
  }
  walk.leave();
}

// The lane's share of one contiguous slice: `on` when the slice is 16-byte aligned on both
// sides and the lane has a whole vector of it; stragglers behind the last whole vector and
// slices that are not aligned are moved here.
__device__ __forceinline__ Move slice_move(uint8_t* d, const uint8_t* s, uint32_t len) {
  const uint32_t tid = threadIdx.x;
  const uintptr_t mis = reinterpret_cast<uintptr_t>(d) | reinterpret_cast<uintptr_t>(s);
  if ((mis & 15u) != 0) {
    copy_slice_odd(d, s, len, tid);
    return KVT_NO_MOVE;
  }
  const uint32_t nvec = len >> 4, done = nvec << 4;
  if (tid < len - done) d[done + tid] = s[done + tid];
  return Move{s, d, tid << 4, tid << 4, tid < nvec};
}

template <bool PACK>
__device__ __forceinline__ Move plain_move(const Item& it) {
  const uint32_t off = it.sub << kSliceShift;
  const uint32_t len = off < it.c.len ? min(kSlice, it.c.len - off) : 0u;  // 0: an idle workgroup
  uint8_t* cache = it.cache + off;
  uint8_t* pk = it.pk + off;
  return slice_move(PACK ? pk : cache, PACK ? cache : pk, len);
}

#define KVT_LAUNCH_STRUCT \
  const Launch L{n_slices, sub_shift & 0xFFu, layer_ptrs, n_tensors, first_layer, n_layers, packed, layer_stride, &blobs, \
                 (sub_shift & kTemporalFlag) != 0, (sub_shift & kCachedStoreFlag) != 0, tickets}

// Gather (PACK) / scatter of a resident chunk table.
template <bool PACK, int MODE>
__global__ __launch_bounds__(kThreads, MODE == kPipelined ? 4 : 8) void copy_chunks_kernel(
    const Chunk* __restrict__ chunks, uint32_t n_slices, uint32_t sub_shift,
    uint8_t* const* __restrict__ layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
    uint32_t n_layers, uint8_t* __restrict__ packed, uint64_t layer_stride, BlobOffsets blobs,
    uint32_t* tickets) {
  KVT_LAUNCH_STRUCT;
  for_items<MODE>(L, [&](uint32_t e) { return fetch_entry(chunks, e); },
                  [&](const Item& it) { return plain_move<PACK>(it); });
}

// The same for a table short enough to be a kernel argument (read through the scalar cache
// like any other argument; the index is uniform across the workgroup).
template <bool PACK, int MODE>
__global__ __launch_bounds__(kThreads, MODE == kPipelined ? 4 : 8) void copy_chunks_small_kernel(
    const SmallTable table, uint32_t n_slices, uint32_t sub_shift,
    uint8_t* const* __restrict__ layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
    uint32_t n_layers, uint8_t* __restrict__ packed, uint64_t layer_stride, BlobOffsets blobs,
    uint32_t* tickets) {
  KVT_LAUNCH_STRUCT;
  for_items<MODE>(L, [&](uint32_t e) { return fetch_entry(table.c, e); },
                  [&](const Item& it) { return plain_move<PACK>(it); });
}

// The capped launch of a plain table whose entries are whole multiples of 16 bytes, 16-byte
// aligned on both sides, and 16 or 32 KiB at most (V = 4 or 8 slices): persistent workgroups
// again, but one table ENTRY per trip -- one descriptor fetch and one pair of buffer
// descriptors for up to 32 KiB, V vectors per lane -- and software-pipelined over three
// register sets: the loads of entry k+1 are issued before the stores of entry k, and a set is
// loaded again only two trips after its stores were issued, so that a wave does not sit out
// the acknowledgement of stores it has just issued (one counter covers a wave's loads and
// stores, in issue order). Lanes beyond an entry's length are switched off by the
// descriptor's range check (loads return zero, stores are dropped), so the loop has no
// branch but its exit. Entries of a layer are dealt to the XCDs in eighths like the slices of
// the other kernels, neighbouring workgroups of an XCD taking neighbouring entries.
typedef __amdgpu_buffer_rsrc_t rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const uint8_t* base, uint32_t bytes) {
  // raw buffer of `bytes` bytes, no stride, no swizzle; 0x00020000: 32-bit data format
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(base), 0, bytes, 0x00020000);
}
// cache-policy operand of the buffer builtins: bit 0 = sc0, bit 1 = nt, bit 4 = sc1
constexpr int kLoadPolicy = 2, kStorePolicy = 1 | 2 | 16;

template <bool PACK, int V, class Fetch>
__device__ __forceinline__ void copy_entries(
    Fetch fetch_table, uint32_t n_chunks, uint8_t* const* __restrict__ layer_ptrs, uint32_t n_tensors,
    uint32_t first_layer, uint32_t n_layers, uint8_t* packed, uint64_t layer_stride,
    const BlobOffsets& blobs, uint32_t* tickets) {
  EntryWalk walk(n_chunks, n_layers, tickets, V == 8 ? 3u : 2u);
  const uint32_t off = threadIdx.x << 4;
  rsrc_t src[3], dst[3];
  u32x4 r[3][V];
  // this workgroup's next entry as two descriptors (empty ones past the end); false past the end
  auto next = [&](int k) -> bool {
    uint32_t item, lay;
    bool valid;
    const bool live = walk.next(item, lay, valid);
    const Entry c = fetch_table(item);
    uint8_t* cache = layer_ptrs[static_cast<uint64_t>(first_layer + lay) * n_tensors + c.tensor()] + c.cache;
    uint8_t* pk = packed + lay * layer_stride + blobs.off[c.tensor()] + c.packed;
    const uint32_t bytes = valid ? c.len : 0u;
    src[k] = make_rsrc(PACK ? cache : pk, bytes);
    dst[k] = make_rsrc(PACK ? pk : cache, bytes);
    return live;
  };
  auto load = [&](int k) {
#pragma unroll
    for (int v = 0; v < V; ++v)
      r[k][v] = __builtin_amdgcn_raw_buffer_load_b128(src[k], off + (v << kSliceShift), 0, kLoadPolicy);
  };
  auto store = [&](int k) {
#pragma unroll
    for (int v = 0; v < V; ++v)
      __builtin_amdgcn_raw_buffer_store_b128(r[k][v], dst[k], off + (v << kSliceShift), 0, kStorePolicy);
  };
  KVT_ROTATE3_PINNED(next, load, store);
  walk.leave();
}

#define KVT_ENTRIES_PARAMS                                                                         \
  uint32_t n_chunks, uint8_t *const *__restrict__ layer_ptrs, uint32_t n_tensors,                  \
      uint32_t first_layer, uint32_t n_layers, uint8_t *packed, uint64_t layer_stride, \
      BlobOffsets blobs, uint32_t *tickets
#define KVT_ENTRIES_ARGS n_chunks, layer_ptrs, n_tensors, first_layer, n_layers, packed, layer_stride, blobs, tickets

template <bool PACK, int V>
__global__ __launch_bounds__(kThreads, 4) void copy_entries_kernel(const Chunk* __restrict__ chunks,
                                                                  KVT_ENTRIES_PARAMS) {
  // read field by field: as one 32-byte load, a gather by fewer workgroups than CUs lost 4-7 %
  const Entry* table = reinterpret_cast<const Entry*>(chunks);
  copy_entries<PACK, V>([&](uint32_t e) { return table[e]; }, KVT_ENTRIES_ARGS);
}
// ... of a table that travels in the kernel arguments
template <bool PACK, int V>
__global__ __launch_bounds__(kThreads, 4) void copy_entries_small_kernel(const SmallTable table,
                                                                        KVT_ENTRIES_PARAMS) {
  copy_entries<PACK, V>([&](uint32_t e) { return entry_of(fetch_entry(table.c, e)); }, KVT_ENTRIES_ARGS);
}

// The same for tables with entries of 4 or 8 KiB (V = 4 or 8 vectors per lane of ONE wavefront):
// with a whole workgroup per entry a lane would hold a single vector or two per trip, and the
// trip's scalar work (walk, table entry, layer pointer, descriptors), which every wavefront
// repeats, would outweigh them. Here a trip takes 4 U entries and wavefront w of the workgroup
// moves the U of them at positions w, w + 4, ... by itself, so it prepares only those.
template <bool PACK, int V, int U, class Fetch>
__device__ __forceinline__ void copy_entries_by_wave(
    Fetch fetch_table, uint32_t n_chunks, uint8_t* const* __restrict__ layer_ptrs, uint32_t n_tensors,
    uint32_t first_layer, uint32_t n_layers, uint8_t* packed, uint64_t layer_stride,
    const BlobOffsets& blobs, uint32_t* tickets) {
  EntryWalk walk(n_chunks, n_layers, tickets, V == 8 ? 1u : 0u);
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t off = (threadIdx.x & 63u) << 4;
  rsrc_t src[3][U], dst[3][U];
  u32x4 r[3][U][V];
  auto next = [&](int k) -> bool {
    bool live = false;
    uint32_t b[4 * U], l[4 * U];
    bool ok[4 * U];
#pragma unroll
    for (int j = 0; j < 4 * U; ++j) {
      const bool more = walk.next(b[j], l[j], ok[j]);
      if (j == 0) live = more;
    }
    uint32_t item[U], lay[U];
    bool valid[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {  // this wavefront's of the trip's entries (uniform selects)
      item[u] = b[4 * u], lay[u] = l[4 * u], valid[u] = ok[4 * u];
#pragma unroll
      for (int w = 1; w < 4; ++w)
        if (wave == static_cast<uint32_t>(w)) item[u] = b[4 * u + w], lay[u] = l[4 * u + w], valid[u] = ok[4 * u + w];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const Entry c = fetch_table(item[u]);
      uint8_t* cache = layer_ptrs[static_cast<uint64_t>(first_layer + lay[u]) * n_tensors + c.tensor()] + c.cache;
      uint8_t* pk = packed + lay[u] * layer_stride + blobs.off[c.tensor()] + c.packed;
      const uint32_t bytes = valid[u] ? c.len : 0u;
      src[k][u] = make_rsrc(PACK ? cache : pk, bytes);
      dst[k][u] = make_rsrc(PACK ? pk : cache, bytes);
    }
    return live;
  };
  auto load = [&](int k) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int v = 0; v < V; ++v)
        r[k][u][v] = __builtin_amdgcn_raw_buffer_load_b128(src[k][u], off + (v << 10), 0, kLoadPolicy);
  };
  auto store = [&](int k) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int v = 0; v < V; ++v)
        __builtin_amdgcn_raw_buffer_store_b128(r[k][u][v], dst[k][u], off + (v << 10), 0, kStorePolicy);
  };
  KVT_ROTATE3_PINNED(next, load, store);
  walk.leave();
}

template <bool PACK, int V, int U>
__global__ __launch_bounds__(kThreads, 4) void copy_entries_by_wave_kernel(const Chunk* __restrict__ chunks,
                                                                          KVT_ENTRIES_PARAMS) {
  const Entry* table = reinterpret_cast<const Entry*>(chunks);
  copy_entries_by_wave<PACK, V, U>([&](uint32_t e) { return table[e]; }, KVT_ENTRIES_ARGS);
}
template <bool PACK, int V, int U>
__global__ __launch_bounds__(kThreads, 4) void copy_entries_by_wave_small_kernel(const SmallTable table,
                                                                                KVT_ENTRIES_PARAMS) {
  copy_entries_by_wave<PACK, V, U>([&](uint32_t e) { return entry_of(fetch_entry(table.c, e)); }, KVT_ENTRIES_ARGS);
}

// The same pipeline for tables whose cache side is not contiguous (strided records, the
// HND <-> NHD transform): one trip moves V slices of one entry (entries of more than V slices
// are taken in parts), the packed side through a descriptor of exactly the part's bytes, the
// cache side through a descriptor that starts at the entry's cache position with the lane's own
// byte offsets, computed when the part is fetched. `cache_offsets(entry, begin, bytes, off)`
// fills the lane's V offsets for the vectors at packed offsets begin + lane * 16 + v * 4096,
// kNoVector where that lies beyond `bytes`. Offsets are 32-bit: the launcher's caller checks
// that no entry spans 2 GiB on the cache side.
constexpr uint32_t kCacheWindow = 0x80000000u;  // bytes a cache-side descriptor covers
constexpr uint32_t kNoVector = kCacheWindow;    // first offset outside it: loads give zero, stores are dropped

template <bool PACK, int V, class CacheOffsets>
__device__ __forceinline__ void entries_pipeline(
    const Chunk* __restrict__ chunks, uint32_t n_chunks, uint32_t part_shift,
    uint8_t* const* __restrict__ layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
    uint32_t n_layers, uint8_t* __restrict__ packed, uint64_t layer_stride,
    const BlobOffsets& blobs, uint32_t* tickets, CacheOffsets cache_offsets) {
  EntryWalk walk(n_chunks << part_shift, n_layers, tickets, V == 8 ? 3u : (V == 4 ? 2u : 1u));
  const uint32_t lane = threadIdx.x << 4;
  const Entry* table = reinterpret_cast<const Entry*>(chunks);
  rsrc_t cdesc[3], pdesc[3];
  uint32_t coff[3][V];
  u32x4 r[3][V];
  auto next = [&](int k) -> bool {
    uint32_t item, lay;
    bool valid;
    const bool live = walk.next(item, lay, valid);
    const Entry c = table[item >> part_shift];
    const uint32_t begin = (item & ((1u << part_shift) - 1u)) * (static_cast<uint32_t>(V) << kSliceShift);
    uint8_t* cache = layer_ptrs[static_cast<uint64_t>(first_layer + lay) * n_tensors + c.tensor()] + c.cache;
    uint8_t* pk = packed + lay * layer_stride + blobs.off[c.tensor()] + c.packed + begin;
    const uint32_t bytes =
        valid && c.len > begin ? min(c.len - begin, static_cast<uint32_t>(V) << kSliceShift) : 0u;
    pdesc[k] = make_rsrc(pk, bytes);
    cdesc[k] = make_rsrc(cache, bytes ? kCacheWindow : 0u);
    cache_offsets(c, begin, bytes, coff[k]);
    return live;
  };
  auto load = [&](int k) {
#pragma unroll
    for (int v = 0; v < V; ++v)
      r[k][v] = PACK ? __builtin_amdgcn_raw_buffer_load_b128(cdesc[k], coff[k][v], 0, kLoadPolicy)
                     : __builtin_amdgcn_raw_buffer_load_b128(pdesc[k], lane + (v << kSliceShift), 0, kLoadPolicy);
  };
  auto store = [&](int k) {
#pragma unroll
    for (int v = 0; v < V; ++v) {
      if (PACK)
        __builtin_amdgcn_raw_buffer_store_b128(r[k][v], pdesc[k], lane + (v << kSliceShift), 0, kStorePolicy);
      else
        __builtin_amdgcn_raw_buffer_store_b128(r[k][v], cdesc[k], coff[k][v], 0, kStorePolicy);
    }
  };
  KVT_ROTATE3(next, load, store);
  walk.leave();
}

// Strided tables (16-byte vectors only; every entry 16-byte aligned on both sides). The
// entry's record shape arrives as one 64-byte scalar load and the offsets are computed without
// a branch: a contiguous entry (shape 0) is the degenerate record whose quotient is always
// zero, so that its vectors are all "column" (both multipliers zero), and a divisor of 1,
// which has no 32-bit reciprocal, adds the dividend itself instead.
typedef uint32_t u32x16 __attribute__((ext_vector_type(16)));
// The lane's V cache-side offsets for the vectors at packed offsets begin + lane + (v << VSHIFT)
// of a strided (or, shape 0, contiguous) entry.
template <bool PACK, int V, int VSHIFT>
__device__ __forceinline__ void strided_offsets(const StrideTable& shapes, const Entry& c, uint32_t begin,
                                                uint32_t bytes, uint32_t lane, uint32_t* coff) {
  const bool plain = c.shape == 0;
  const u32x16 raw = *reinterpret_cast<const u32x16*>(&shapes.shape[plain ? 0u : c.shape - 1u]);
  // words of a StrideShape: 0 vlen, 1 inv_vlen, 2 n_inner, 4 + 2 side: outer, 8 + 2 side: inner,
  // 12 inv_inner (low halves of the strides: the entry spans less than 2 GiB)
  const uint32_t vlen = plain ? 0u : raw[0];
  const uint32_t rec_mul = plain || raw[0] == 1u ? 0u : raw[1], rec_add = !plain && raw[0] == 1u ? 1u : 0u;
  const uint32_t n_inner = plain ? 1u : raw[2];
  const uint32_t o_mul = raw[12], o_add = n_inner == 1u ? 1u : 0u;
  const uint32_t outer = raw[PACK ? 4 : 6], inner = raw[PACK ? 8 : 10];
#pragma unroll
  for (int v = 0; v < V; ++v) {
    const uint32_t at = lane + (v << VSHIFT);
    const uint32_t vi = (begin + at) >> 4;  // vector index inside the entry, < 2^15
    const uint32_t rec = __umulhi(vi, rec_mul) + vi * rec_add;
    const uint32_t col = vi - rec * vlen;
    const uint32_t o = __umulhi(rec, o_mul) + rec * o_add;
    const uint32_t i = rec - o * n_inner;
    coff[v] = at < bytes ? o * outer + i * inner + (col << 4) : kNoVector;
  }
}

template <bool PACK, int V>
__global__ __launch_bounds__(kThreads, 4) void strided_entries_kernel(
    const Chunk* __restrict__ chunks, uint32_t n_chunks, uint32_t part_shift,
    uint8_t* const* __restrict__ layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
    uint32_t n_layers, uint8_t* __restrict__ packed, uint64_t layer_stride, BlobOffsets blobs,
    StrideTable shapes, uint32_t* tickets) {
  const uint32_t lane = threadIdx.x << 4;
  entries_pipeline<PACK, V>(
      chunks, n_chunks, part_shift, layer_ptrs, n_tensors, first_layer, n_layers, packed, layer_stride,
      blobs, tickets, [&](const Entry& c, uint32_t begin, uint32_t bytes, uint32_t* coff) {
        strided_offsets<PACK, V, kSliceShift>(shapes, c, begin, bytes, lane, coff);
      });
}

// Strided and transposing tables with entries of 4 or 8 KiB (senders or receivers on TP4 / TP8:
// a block's share of one rank is that small): a wavefront per entry, as in
// copy_entries_by_wave_kernel, with the cache side through a 2 GiB window and per-lane offsets.
// `cache_offsets(entry, bytes, off)` fills the lane's V offsets for the vectors at packed
// offsets lane * 16 + v * 1024 of the entry (lane = lane of the wavefront).
template <bool PACK, int V, int U, class CacheOffsets>
__device__ __forceinline__ void entries_pipeline_by_wave(
    const Chunk* __restrict__ chunks, uint32_t n_chunks, uint8_t* const* __restrict__ layer_ptrs,
    uint32_t n_tensors, uint32_t first_layer, uint32_t n_layers, uint8_t* __restrict__ packed,
    uint64_t layer_stride, const BlobOffsets& blobs, uint32_t* tickets, CacheOffsets cache_offsets) {
  EntryWalk walk(n_chunks, n_layers, tickets, V == 8 ? 1u : 0u);
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t lane = (threadIdx.x & 63u) << 4;
  const Entry* table = reinterpret_cast<const Entry*>(chunks);
  rsrc_t cdesc[3][U], pdesc[3][U];
  uint32_t coff[3][U][V];
  u32x4 r[3][U][V];
  auto next = [&](int k) -> bool {
    bool live = false;
    uint32_t b[4 * U], l[4 * U];
    bool ok[4 * U];
#pragma unroll
    for (int j = 0; j < 4 * U; ++j) {
      const bool more = walk.next(b[j], l[j], ok[j]);
      if (j == 0) live = more;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {  // this wavefront's of the trip's entries (uniform selects)
      uint32_t item = b[4 * u], lay = l[4 * u];
      bool valid = ok[4 * u];
#pragma unroll
      for (int w = 1; w < 4; ++w)
        if (wave == static_cast<uint32_t>(w)) item = b[4 * u + w], lay = l[4 * u + w], valid = ok[4 * u + w];
      const Entry c = table[item];
      uint8_t* cache = layer_ptrs[static_cast<uint64_t>(first_layer + lay) * n_tensors + c.tensor()] + c.cache;
      uint8_t* pk = packed + lay * layer_stride + blobs.off[c.tensor()] + c.packed;
      const uint32_t bytes = valid ? c.len : 0u;
      pdesc[k][u] = make_rsrc(pk, bytes);
      cdesc[k][u] = make_rsrc(cache, bytes ? kCacheWindow : 0u);
      cache_offsets(c, bytes, coff[k][u]);
    }
    return live;
  };
  auto load = [&](int k) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int v = 0; v < V; ++v)
        r[k][u][v] = PACK ? __builtin_amdgcn_raw_buffer_load_b128(cdesc[k][u], coff[k][u][v], 0, kLoadPolicy)
                          : __builtin_amdgcn_raw_buffer_load_b128(pdesc[k][u], lane + (v << 10), 0, kLoadPolicy);
  };
  auto store = [&](int k) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int v = 0; v < V; ++v) {
        if (PACK)
          __builtin_amdgcn_raw_buffer_store_b128(r[k][u][v], pdesc[k][u], lane + (v << 10), 0, kStorePolicy);
        else
          __builtin_amdgcn_raw_buffer_store_b128(r[k][u][v], cdesc[k][u], coff[k][u][v], 0, kStorePolicy);
      }
  };
  KVT_ROTATE3(next, load, store);
  walk.leave();
}

#define KVT_BY_WAVE_PARAMS                                                                            \
  const Chunk *__restrict__ chunks, uint32_t n_chunks, uint8_t *const *__restrict__ layer_ptrs,        \
      uint32_t n_tensors, uint32_t first_layer, uint32_t n_layers, uint8_t *__restrict__ packed,       \
      uint64_t layer_stride, BlobOffsets blobs
#define KVT_BY_WAVE_ARGS chunks, n_chunks, layer_ptrs, n_tensors, first_layer, n_layers, packed, layer_stride, blobs

template <bool PACK, int V, int U>
__global__ __launch_bounds__(kThreads, 4) void strided_entries_by_wave_kernel(KVT_BY_WAVE_PARAMS,
                                                                             StrideTable shapes,
                                                                             uint32_t* tickets) {
  const uint32_t lane = (threadIdx.x & 63u) << 4;
  entries_pipeline_by_wave<PACK, V, U>(KVT_BY_WAVE_ARGS, tickets,
                                       [&](const Entry& c, uint32_t bytes, uint32_t* coff) {
                                         strided_offsets<PACK, V, 10>(shapes, c, 0u, bytes, lane, coff);
                                       });
}

// The HND <-> NHD transform (index arithmetic of xform_chunks_kernel): the lane's V cache-side
// offsets for the vectors at packed offsets begin + lane + (v << VSHIFT) of an entry.
template <int V, int VSHIFT>
__device__ __forceinline__ void xform_offsets(const XformDev& x, const Entry& c, uint32_t begin,
                                              uint32_t bytes, uint32_t lane, uint32_t* coff) {
#pragma unroll
  for (int v = 0; v < V; ++v) {
    const uint32_t at = lane + (v << VSHIFT);
    const uint32_t vi = (begin + at) >> 4;
    const uint32_t r = x.vrow == 1 ? vi : __umulhi(vi, x.inv_vrow);
    const uint32_t col = vi - r * x.vrow;
    const uint32_t t_local = x.heads == 1 ? r : __umulhi(r, x.inv_heads);
    const uint32_t h = r - t_local * x.heads;
    const uint32_t cidx = (h * x.ntpb + c.t0() + t_local) * x.vrow + col;
    coff[v] = at < bytes ? cidx << 4 : kNoVector;
  }
}

template <bool PACK, int V>
__global__ __launch_bounds__(kThreads, 4) void xform_entries_kernel(
    const Chunk* __restrict__ chunks, uint32_t n_chunks, uint32_t part_shift,
    uint8_t* const* __restrict__ layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
    uint32_t n_layers, uint8_t* __restrict__ packed, uint64_t layer_stride, BlobOffsets blobs,
    XformDev x, uint32_t* tickets) {
  const uint32_t lane = threadIdx.x << 4;
  entries_pipeline<PACK, V>(
      chunks, n_chunks, part_shift, layer_ptrs, n_tensors, first_layer, n_layers, packed, layer_stride,
      blobs, tickets, [&](const Entry& c, uint32_t begin, uint32_t bytes, uint32_t* coff) {
        xform_offsets<V, kSliceShift>(x, c, begin, bytes, lane, coff);
      });
}

template <bool PACK, int V, int U>
__global__ __launch_bounds__(kThreads, 4) void xform_entries_by_wave_kernel(KVT_BY_WAVE_PARAMS, XformDev x,
                                                                           uint32_t* tickets) {
  const uint32_t lane = (threadIdx.x & 63u) << 4;
  entries_pipeline_by_wave<PACK, V, U>(KVT_BY_WAVE_ARGS, tickets,
                                       [&](const Entry& c, uint32_t bytes, uint32_t* coff) {
                                         xform_offsets<V, 10>(x, c, 0u, bytes, lane, coff);
                                       });
}

// Gather / scatter of a table whose chunks may be strided on the cache side:
// the token -> offset arithmetic of the TP-remapping layouts (one short range
// per token, per head, K and V) is evaluated here, per 16-byte vector, instead
// of being materialised as one table entry per range. Contiguous chunks
// (shape 0) take the plain path. Cache offsets, strides and record lengths of
// strided chunks are multiples of 16 by construction; WORDS = false additionally
// needs 16-byte aligned base pointers and blob positions (one vector per lane),
// WORDS = true moves 4-byte words instead (a blob inside a received layer
// message sits at 4 or 12 modulo 16; that path is PCIe-bound anyway).
template <bool PACK, bool WORDS, bool CAPPED>
__global__ __launch_bounds__(kThreads, 8) void strided_chunks_kernel(
    const Chunk* __restrict__ chunks, uint32_t n_slices, uint32_t sub_shift,
    uint8_t* const* __restrict__ layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
    uint32_t n_layers, uint8_t* __restrict__ packed, uint64_t layer_stride, BlobOffsets blobs,
    StrideTable shapes, uint32_t* tickets) {
  KVT_LAUNCH_STRUCT;
  for_items<CAPPED ? kStriding : kOnePerSlice>(L, [&](uint32_t e) { return fetch_entry(chunks, e); }, [&](const Item& it) -> Move {
    if (it.c.shape == 0) return plain_move<PACK>(it);
    const uint32_t off = it.sub << kSliceShift;
    if (off >= it.c.len) return KVT_NO_MOVE;
    const uint32_t len = min(kSlice, it.c.len - off);
    uint8_t* cache = it.cache;
    uint8_t* pk = it.pk + off;
    const StrideShape& s = shapes.shape[it.c.shape - 1u];
    const uint64_t outer = s.outer[PACK ? 0 : 1], inner = s.inner[PACK ? 0 : 1];
    if (!WORDS) {
      const uint32_t v = (off >> 4) + threadIdx.x;  // vector index inside the chunk, < 2^15
      const uint32_t rec = s.vlen == 1 ? v : __umulhi(v, s.inv_vlen);
      const uint32_t col = v - rec * s.vlen;
      const uint32_t o = s.n_inner == 1 ? rec : (s.n_inner == 2 ? rec >> 1 : rec / s.n_inner);
      const uint32_t i = rec - o * s.n_inner;
      const uint64_t cv = o * outer + i * inner + (col << 4), pv = threadIdx.x << 4;
      return Move{PACK ? cache : pk, PACK ? pk : cache, PACK ? cv : pv, PACK ? pv : cv,
                  threadIdx.x < (len >> 4)};
    }
    const uint32_t wlen = s.vlen << 2;  // record length in words, < 1024
#pragma clang loop vectorize(disable) unroll(disable)
    for (uint32_t t = threadIdx.x; t < (len >> 2); t += kThreads) {
      const uint32_t w = (off >> 2) + t;          // word index inside the chunk, < 2^17
      const uint32_t rec = __umulhi(w, s.inv_wlen);
      const uint32_t col = w - rec * wlen;
      const uint32_t o = s.n_inner == 1 ? rec : (s.n_inner == 2 ? rec >> 1 : rec / s.n_inner);
      const uint32_t i = rec - o * s.n_inner;
      uint32_t* cw = reinterpret_cast<uint32_t*>(cache + o * outer + i * inner + (col << 2));
      uint32_t* pw = reinterpret_cast<uint32_t*>(pk) + t;
      if (PACK)
        *pw = *cw;
      else
        *cw = *pw;
    }
    return KVT_NO_MOVE;
  });
}

// HND <-> NHD page transform. A chunk covers tokens [t0, t0 + len/(heads*row))
// of one K or V half page whose base is c.cache. Packed side: [token][head][row]
// contiguous from c.packed; cache side: [head][ntpb][row]. Lane v of the chunk
// moves the v-th 16-byte vector of the packed side; a row is vrow vectors.
template <bool PACK, bool CAPPED>
__global__ __launch_bounds__(kThreads, 8) void xform_chunks_kernel(
    const Chunk* __restrict__ chunks, uint32_t n_slices, uint32_t sub_shift,
    uint8_t* const* __restrict__ layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
    uint32_t n_layers, uint8_t* __restrict__ packed, uint64_t layer_stride, BlobOffsets blobs,
    XformDev x, uint32_t* tickets) {
  KVT_LAUNCH_STRUCT;
  for_items<CAPPED ? kStriding : kOnePerSlice>(L, [&](uint32_t e) { return fetch_entry(chunks, e); }, [&](const Item& it) -> Move {
    const uint32_t v = (it.sub << 8) + threadIdx.x;  // 256 vectors per slice
    // exact quotients by multiply-high (operands < 2^16); a divisor of 1 has no such constant
    const uint32_t r = x.vrow == 1 ? v : __umulhi(v, x.inv_vrow);  // packed-side row: t_local*heads + h
    const uint32_t col = v - r * x.vrow;
    const uint32_t t_local = x.heads == 1 ? r : __umulhi(r, x.inv_heads);
    const uint32_t h = r - t_local * x.heads;
    const uint32_t cidx = (h * x.ntpb + it.c.t0() + t_local) * x.vrow + col;
    const uint64_t cv = static_cast<uint64_t>(cidx) << 4, pv = v << 4;
    return Move{PACK ? it.cache : it.pk, PACK ? it.pk : it.cache, PACK ? cv : pv, PACK ? pv : cv,
                v < (it.c.len >> 4)};
  });
}

// Range-granular copy driven by three int64 device arrays (the reference's
// launcher interface). blockIdx.y strides over ranges; the gridDim.x workgroups
// ("rows") of one range stride over its 4 KiB slices. Rows are the fast grid
// dimension, so workgroups dispatched together work on neighbouring slices of
// the same range (measured against ranges-fast order: +1 to +3 %).
__global__ __launch_bounds__(kThreads) void copy_ranges_kernel(
    const uint8_t* __restrict__ src_base, uint8_t* __restrict__ dst_base,
    const int64_t* __restrict__ src_off, const int64_t* __restrict__ dst_off,
    const int64_t* __restrict__ lens, int64_t n) {
  for (int64_t i = blockIdx.y; i < n; i += gridDim.y) {
    const uint64_t len = static_cast<uint64_t>(lens[i]);
    const uint8_t* s = src_base + src_off[i];
    uint8_t* d = dst_base + dst_off[i];
    for (uint64_t o = static_cast<uint64_t>(blockIdx.x) << kSliceShift; o < len;
         o += static_cast<uint64_t>(gridDim.x) << kSliceShift) {
      const uint64_t m = len - o;
      copy_slice(d + o, s + o, static_cast<uint32_t>(m < kSlice ? m : kSlice), threadIdx.x);
    }
  }
}

// The same list under a CU-share limit: persistent workgroups whose wavefronts each walk ranges
// of their own (the ranges are dealt to the XCDs in eighths, the wavefronts of an XCD stride
// through its eighth), 8 KiB of a range per trip through range-checked buffer descriptors,
// software-pipelined over three register sets like copy_entries_by_wave_kernel. With one
// vector per lane in flight (copy_ranges_kernel on a limited grid) the rate follows the wave
// slots: 4.7 TB/s at a quarter of the device, 2.7 at an eighth. Lengths and addresses live on
// the device, so alignment is found out here: a range that is not 4-byte aligned on both sides
// is copied by its wavefront on the spot, and so are the bytes behind the last whole vector of
// an aligned one (16-byte buffer accesses need 4-byte alignment only; ranges 4 bytes off on one
// side: 4.6-5.0 TB/s against 4.0-4.4 on the grid, which moves them as words).
// (4-byte words where both sides allow it, else bytes; sixteen loads in flight per lane)
template <class T>
__device__ __forceinline__ void copy_units_by_wave(T* d, const T* s, uint64_t count, uint32_t lane) {
  constexpr int kInFlight = 16;
#pragma clang loop unroll(disable)
  for (uint64_t base = 0; base < count; base += 64u * kInFlight) {
    T v[kInFlight];
#pragma unroll
    for (int j = 0; j < kInFlight; ++j) {
      const uint64_t i = base + lane + 64u * j;
      v[j] = i < count ? __builtin_nontemporal_load(s + i) : T(0);
    }
#pragma unroll
    for (int j = 0; j < kInFlight; ++j) {
      const uint64_t i = base + lane + 64u * j;
      if (i < count) __builtin_nontemporal_store(v[j], d + i);
    }
  }
}
__device__ __forceinline__ void copy_range_odd_by_wave(uint8_t* d, const uint8_t* s, uint64_t len, uint32_t lane) {
  if (((reinterpret_cast<uintptr_t>(s) | reinterpret_cast<uintptr_t>(d)) & 3u) == 0) {
    const uint64_t words = len >> 2;
    copy_units_by_wave(reinterpret_cast<uint32_t*>(d), reinterpret_cast<const uint32_t*>(s), words, lane);
    const uint64_t done = words << 2;
    if (lane < len - done) d[done + lane] = s[done + lane];
  } else {
    copy_units_by_wave(d, s, len, lane);
  }
}
// A wavefront's unit of work is a whole range, so one very long range among short ones (a merged
// run of hundreds of blocks) would be moved by a single wavefront long after the others have
// left. With a block of its own (`share`: word 0 the number of listed ranges, word 1 the
// wavefronts that have left the second kernel, from word 2 the listed indices; all zero
// between launches) the wavefront that meets a range above kLongRange lists it instead of
// moving it (when the list is full it moves it after all), and move_listed_ranges_kernel,
// launched behind, moves the listed ranges with every wavefront, in segments of kSegment dealt
// out by position: the segments are numbered through all listed ranges and a wavefront takes
// those whose number is its own modulo the wavefronts. The last wavefront to leave zeroes the
// words used.
constexpr uint32_t kSegment = 64u << 10;
static_assert((2 + kShareMax) * 4 <= kShareBlockBytes, "the list of long ranges must fit its block");
__global__ __launch_bounds__(kThreads, 2) void move_listed_ranges_kernel(
    const uint8_t* src_base, uint8_t* dst_base, const int64_t* __restrict__ src_off,
    const int64_t* __restrict__ dst_off, const int64_t* __restrict__ lens, uint32_t* share) {
  const uint32_t listed = __builtin_amdgcn_readfirstlane(share[0]);
  if (listed == 0) return;  // (every wavefront sees the same: nobody counts itself out below)
  const uint32_t n_long = listed < kShareMax ? listed : kShareMax;
  constexpr uint32_t kTrip = 8u << 10, kNoSegment = 0xFFFFFFFFu;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t lane64 = threadIdx.x & 63u, off = lane64 << 4;
  const uint32_t walkers = gridDim.x * 4u, me = blockIdx.x * 4u + wave;
  const uint32_t* list = share + 2;
  // j: the listed range the wavefront is at; before: the segments of the ranges in front of it
  // (mod walkers); seg: its next segment in range j (kNoSegment: not worked out yet)
  uint32_t j = 0, before = 0, seg = kNoSegment;
  const uint8_t* s = nullptr;
  uint8_t* d = nullptr;
  uint64_t len = 0, begin = 0;
  rsrc_t src[3], dst[3];
  u32x4 r[3][8];
  auto next = [&](int k) -> bool {
    bool live = true;
    if (begin >= len) {
      len = 0;
      begin = 0;
      live = false;
      uint32_t odd = 0;
      while (j < n_long) {
        const uint32_t at = __builtin_amdgcn_readfirstlane(list[j]);
        const uint64_t whole = static_cast<uint64_t>(lens[at]);
        const uint64_t n_seg = (whole + kSegment - 1) / kSegment;
        if (seg == kNoSegment) seg = __builtin_amdgcn_readfirstlane((me + walkers - before) % walkers);
        if (seg < n_seg) {
          const uint64_t o = static_cast<uint64_t>(seg) * kSegment;
          const uint64_t l = whole - o < kSegment ? whole - o : kSegment;
          s = src_base + src_off[at] + o;
          d = dst_base + dst_off[at] + o;
          if (((reinterpret_cast<uintptr_t>(s) | reinterpret_cast<uintptr_t>(d)) & 3u) == 0) {
            len = l & ~15ull;  // whole vectors through the pipeline, the last bytes at once
            if (lane64 < (l & 15u)) d[len + lane64] = s[len + lane64];
          } else {
            odd = static_cast<uint32_t>(l);
          }
          seg += walkers;
          live = true;
          break;
        }
        before = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>((before + n_seg) % walkers));
        seg = kNoSegment;
        ++j;
      }
      // a segment that is not 4-byte aligned on both sides: byte by byte, on the spot
#pragma unroll 8
      for (uint32_t b = lane64; b < odd; b += 64u) d[b] = s[b];
    }
    const uint64_t left = len - begin;
    const uint32_t bytes = left < kTrip ? static_cast<uint32_t>(left) : kTrip;
    src[k] = make_rsrc(s + begin, bytes);
    dst[k] = make_rsrc(d + begin, bytes);
    begin += bytes;
    return live;
  };
  auto load = [&](int k) {
#pragma unroll
    for (int v = 0; v < 8; ++v)
      r[k][v] = __builtin_amdgcn_raw_buffer_load_b128(src[k], off + (v << 10), 0, kLoadPolicy);
  };
  auto store = [&](int k) {
#pragma unroll
    for (int v = 0; v < 8; ++v)
      __builtin_amdgcn_raw_buffer_store_b128(r[k][v], dst[k], off + (v << 10), 0, kStorePolicy);
  };
  KVT_ROTATE3_PINNED(next, load, store);
  uint32_t left = 0;
  if (lane64 == 0) left = atomicAdd(share + 1, 1u);
  if (static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(left)) == walkers - 1u)  // the last wavefront out
    for (uint32_t w = lane64; w < 2u + n_long; w += 64u) share[w] = 0;
}
template <int U>
__global__ __launch_bounds__(kThreads, 4) void copy_ranges_persistent_kernel(
    const uint8_t* src_base, uint8_t* dst_base, const int64_t* __restrict__ src_off,
    const int64_t* __restrict__ dst_off, const int64_t* __restrict__ lens, uint32_t n,
    uint32_t* share) {
  // U ranges at a time per wavefront, each in trips of 8 / U KiB: the same bytes in flight, and
  // more ranges a second where they are short, since a range costs a trip however short it is
  // (TB/s with 1 / 2 / 4: ranges of 256 B 0.55 / 0.92 / 1.42, of 1 KiB 2.1 / 3.3 / 4.8, of 4 KiB
  // 5.4 / 6.1 / 5.4, of 16 KiB 6.4 / 6.3 / 5.6)
  constexpr int V = 8 / U;
  constexpr uint32_t kTrip = static_cast<uint32_t>(V) << 10;  // bytes of a range per trip
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t lane64 = threadIdx.x & 63u, off = lane64 << 4;
  const uint32_t per8 = (n + 7u) >> 3, xcd = blockIdx.x & 7u;
  const uint32_t step = (gridDim.x >> 3) * 4u * U;   // range walkers per XCD
  uint32_t within[U];                                 // each walker's next range inside the eighth
  const uint8_t* s[U];
  uint8_t* d[U];
  uint64_t len[U], begin[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    within[u] = ((blockIdx.x >> 3) * 4u + wave) * U + u;
    s[u] = nullptr, d[u] = nullptr, len[u] = 0, begin[u] = 0;
  }
  rsrc_t src[3][U], dst[3][U];
  u32x4 r[3][U][V];
  // the walker's current range is (s, d, l): whole vectors through the pipeline, the last bytes
  // and a range that is not 4-byte aligned on the spot
  auto begin_range = [&](int u, uint64_t l) {
    if (((reinterpret_cast<uintptr_t>(s[u]) | reinterpret_cast<uintptr_t>(d[u])) & 3u) == 0) {
      len[u] = l & ~15ull;
      if (lane64 < (l & 15u)) d[u][len[u] + lane64] = s[u][len[u] + lane64];
    } else {
      copy_range_odd_by_wave(d[u], s[u], l, lane64);
    }
  };
  auto trip = [&](int k, int u) {
    const uint64_t left = len[u] - begin[u];  // 0 when there is nothing (more) to move: empty descriptors
    const uint32_t bytes = left < kTrip ? static_cast<uint32_t>(left) : kTrip;
    src[k][u] = make_rsrc(s[u] + begin[u], bytes);
    dst[k][u] = make_rsrc(d[u] + begin[u], bytes);
    begin[u] += bytes;
  };
  auto next = [&](int k) -> bool {
    bool any = false;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      bool live = true;
      if (begin[u] >= len[u]) {  // on to the next range
        const uint32_t i = xcd * per8 + within[u];
        live = within[u] < per8 && i < n;
        within[u] += step;
        len[u] = 0;
        begin[u] = 0;
        if (live) {
          const uint64_t l = static_cast<uint64_t>(lens[i]);
          s[u] = src_base + src_off[i];
          d[u] = dst_base + dst_off[i];
          bool mine = true;
          if (share && l > kLongRange) {  // everybody's, later, if the list has room
            uint32_t at = 0;
            if (lane64 == 0) at = atomicAdd(share, 1u);
            at = __builtin_amdgcn_readfirstlane(at);
            mine = at >= kShareMax;
            if (!mine && lane64 == 0) share[2 + at] = i;
          }
          if (mine) begin_range(u, l);
        }
      }
      trip(k, u);
      any = any || live;
    }
    return any;
  };
  auto load = [&](int k) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int v = 0; v < V; ++v)
        r[k][u][v] = __builtin_amdgcn_raw_buffer_load_b128(src[k][u], off + (v << 10), 0, kLoadPolicy);
  };
  auto store = [&](int k) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int v = 0; v < V; ++v)
        __builtin_amdgcn_raw_buffer_store_b128(r[k][u][v], dst[k][u], off + (v << 10), 0, kStorePolicy);
  };
  KVT_ROTATE3_PINNED(next, load, store);
}

// bf16 -> fp8 E4M3 (OCP "fn" variant: no infinities, 0x7F = NaN), round to
// nearest even, finite values and infinities saturate to +-448 (0x7E), NaN
// stays NaN (sign kept). `pair` holds two bf16; the two fp8 bytes go to the low
// (HIGH = false) or high half of `acc`. The matrix-core conversion instruction
// of gfx950 rounds exactly like the integer definition (checked for all 65 536
// bit patterns by the tests); its overflow result depends on a mode bit, so the
// operands are clamped to +-448 first, and NaNs, which the clamp would turn
// into 448, are patched afterwards.
template <bool HIGH>
__device__ __forceinline__ uint32_t bf16x2_to_e4m3(uint32_t pair, uint32_t acc) {
  const float a = __uint_as_float(pair << 16);
  const float b = __uint_as_float(pair & 0xFFFF0000u);
  uint32_t r = __builtin_amdgcn_cvt_pk_fp8_f32(__builtin_amdgcn_fmed3f(a, -448.0f, 448.0f),
                                               __builtin_amdgcn_fmed3f(b, -448.0f, 448.0f), acc, HIGH);
  constexpr uint32_t sh = HIGH ? 16u : 0u;
  if (a != a) r = (r & ~(0xFFu << sh)) | ((((pair >> 8) & 0x80u) | 0x7Fu) << sh);
  if (b != b) r = (r & ~(0xFF00u << sh)) | ((((pair >> 24) & 0x80u) | 0x7Fu) << (sh + 8u));
  return r;
}

__device__ __forceinline__ uint32_t cvt4(uint32_t lo, uint32_t hi) {
  return bf16x2_to_e4m3<true>(hi, bf16x2_to_e4m3<false>(lo, 0u));
}

// One element (stragglers of a range).
__device__ __forceinline__ uint32_t bf16_to_e4m3(uint32_t bits) {
  return bf16x2_to_e4m3<false>(bits & 0xFFFFu, 0u) & 0xFFu;
}

// Converting gather: range i = lens[i] bf16 elements at src_base + src_off[i]
// -> lens[i] fp8 bytes at dst_base + dst_off[i]. A slice is 4096 elements
// (8 KiB in, 4 KiB out): two groups of 8 elements per lane. Grid as in copy_ranges_kernel.
__global__ __launch_bounds__(kThreads) void convert_ranges_kernel(
    const uint8_t* __restrict__ src_base, uint8_t* __restrict__ dst_base,
    const int64_t* __restrict__ src_off, const int64_t* __restrict__ dst_off,
    const int64_t* __restrict__ lens, int64_t n) {
  for (int64_t i = blockIdx.y; i < n; i += gridDim.y) {
    const uint64_t count = static_cast<uint64_t>(lens[i]);
    const uint8_t* s_range = src_base + src_off[i];
    uint8_t* d_range = dst_base + dst_off[i];
    const bool aligned =
        ((reinterpret_cast<uintptr_t>(s_range) | reinterpret_cast<uintptr_t>(d_range)) & 15u) == 0;
    for (uint64_t o = static_cast<uint64_t>(blockIdx.x) << kSliceShift; o < count;
         o += static_cast<uint64_t>(gridDim.x) << kSliceShift) {
      const uint32_t m = static_cast<uint32_t>(count - o < kSlice ? count - o : kSlice);
      const uint8_t* s8 = s_range + 2 * o;
      uint8_t* d8 = d_range + o;
      uint32_t done = 0;
      if (aligned) {
        // groups of 8 elements (16 bytes in, 8 bytes out); lane t takes groups t and t + 256,
        // so that loads and stores are contiguous across the wavefront
        typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
        const uint32_t n_groups = m >> 3;
        u32x4 in[2];
#pragma unroll
        for (int k = 0; k < 2; ++k) {
          const uint32_t g = threadIdx.x + (k << 8);
          in[k] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(s8) + (g < n_groups ? g : 0u));
        }
#pragma unroll
        for (int k = 0; k < 2; ++k) {
          const uint32_t g = threadIdx.x + (k << 8);
          if (g >= n_groups) continue;
          u32x2 r;
          r.x = cvt4(in[k].x, in[k].y);
          r.y = cvt4(in[k].z, in[k].w);
          __builtin_nontemporal_store(r, reinterpret_cast<u32x2*>(d8) + g);
        }
        done = n_groups << 3;
      }
      const uint16_t* s16 = reinterpret_cast<const uint16_t*>(s8);
      for (uint32_t j = done + threadIdx.x; j < m; j += kThreads)
        d8[j] = static_cast<uint8_t>(bf16_to_e4m3(s16[j]));
    }
  }
}

// The converting gather by persistent workgroups, a wavefront per range (see
// copy_ranges_persistent_kernel): 4096 elements of a range per trip, lane t of the wavefront
// the groups of 8 elements t, t + 64, ... t + 448. A range that is not 4-byte aligned on both
// sides is converted by its wavefront on the spot, element-wise, and so are the elements behind
// the last whole group of an aligned one.
__global__ __launch_bounds__(kThreads, 4) void convert_ranges_persistent_kernel(
    const uint8_t* src_base, uint8_t* dst_base, const int64_t* __restrict__ src_off,
    const int64_t* __restrict__ dst_off, const int64_t* __restrict__ lens, uint32_t n) {
  constexpr int G = 8;
  constexpr uint32_t kTrip = static_cast<uint32_t>(G) << 9;  // elements of a range per trip
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t lane64 = threadIdx.x & 63u;
  const uint32_t per8 = (n + 7u) >> 3, xcd = blockIdx.x & 7u;
  const uint32_t step = (gridDim.x >> 3) * 4u;
  uint32_t within = (blockIdx.x >> 3) * 4u + wave;
  const uint8_t* s = nullptr;
  uint8_t* d = nullptr;
  uint64_t count = 0, begin = 0;
  rsrc_t src[3], dst[3];
  u32x4 r[3][G];
  auto next = [&](int k) -> bool {
    bool live = true;
    if (begin >= count) {  // on to the next range
      const uint32_t i = xcd * per8 + within;
      live = within < per8 && i < n;
      within += step;
      count = 0;
      begin = 0;
      if (live) {
        const uint64_t c = static_cast<uint64_t>(lens[i]);
        s = src_base + src_off[i];
        d = dst_base + dst_off[i];
        const uint16_t* s16 = reinterpret_cast<const uint16_t*>(s);
        if (((reinterpret_cast<uintptr_t>(s) | reinterpret_cast<uintptr_t>(d)) & 3u) == 0) {
          count = c & ~7ull;  // whole groups through the pipeline, the last elements at once
          if (lane64 < (c & 7u)) d[count + lane64] = static_cast<uint8_t>(bf16_to_e4m3(s16[count + lane64]));
        } else {
#pragma clang loop vectorize(disable) unroll(disable)
          for (uint64_t j = lane64; j < c; j += 64) d[j] = static_cast<uint8_t>(bf16_to_e4m3(s16[j]));
        }
      }
    }
    const uint64_t left = count - begin;
    const uint32_t elems = left < kTrip ? static_cast<uint32_t>(left) : kTrip;
    src[k] = make_rsrc(s + 2 * begin, 2 * elems);
    dst[k] = make_rsrc(d + begin, elems);
    begin += elems;
    return live;
  };
  auto load = [&](int k) {
#pragma unroll
    for (int j = 0; j < G; ++j)
      r[k][j] = __builtin_amdgcn_raw_buffer_load_b128(src[k], (lane64 + (j << 6)) << 4, 0, kLoadPolicy);
  };
  auto store = [&](int k) {
#pragma unroll
    for (int j = 0; j < G; ++j) {
      u32x2 out;
      out.x = cvt4(r[k][j].x, r[k][j].y);
      out.y = cvt4(r[k][j].z, r[k][j].w);
      __builtin_amdgcn_raw_buffer_store_b64(out, dst[k], (lane64 + (j << 6)) << 3, 0, kStorePolicy);
    }
  };
  KVT_ROTATE3_PINNED(next, load, store);
}

// Converting gather of a resident chunk table (the pack direction of a plan whose source
// cache holds bf16 and whose transfer buffer and destination hold fp8): chunk lengths,
// packed positions and record lengths count fp8 bytes, i.e. elements; cache offsets and
// strides count bytes of the bf16 cache, so element e of a contiguous piece is read at byte
// 2e. One workgroup converts 4096 elements (8 KiB in, 4 KiB out), two groups of 8 per lane. Strided
// chunks (shape != 0) are 16-byte aligned on both sides by construction.
template <bool CAPPED>
__global__ __launch_bounds__(kThreads, 8) void convert_chunks_kernel(
    const Chunk* __restrict__ chunks, uint32_t n_slices, uint32_t sub_shift,
    uint8_t* const* __restrict__ layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
    uint32_t n_layers, uint8_t* __restrict__ packed, uint64_t layer_stride, BlobOffsets blobs,
    StrideTable shapes, uint32_t* tickets) {
  KVT_LAUNCH_STRUCT;
  // a conversion between load and store: `place` moves everything itself. A slice is 4096
  // elements = 512 groups of 8 (16 bytes in, 8 bytes out); lane t takes groups t and t + 256, so
  // that both of its loads and both of its stores are contiguous across the wavefront (a lane
  // that loads 32 contiguous bytes makes every load touch twice the lines it uses: measured
  // 2.7 % slower on the TP2 -> TP1 batch).
  for_items<CAPPED ? kStriding : kOnePerSlice>(L, [&](uint32_t e) { return fetch_entry(chunks, e); }, [&](const Item& it) -> Move {
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const uint32_t off = it.sub << kSliceShift;
    if (off >= it.c.len) return KVT_NO_MOVE;
    const uint32_t len = min(kSlice, it.c.len - off);
    const uint8_t* cache = it.cache;
    uint8_t* pk = it.pk + off;
    if (it.c.shape == 0) {
      const uint8_t* s8 = cache + 2ull * off;
      if (((reinterpret_cast<uintptr_t>(s8) | reinterpret_cast<uintptr_t>(pk)) & 15u) != 0) {
        const uint16_t* s16 = reinterpret_cast<const uint16_t*>(s8);
        for (uint32_t j = threadIdx.x; j < len; j += kThreads)
          pk[j] = static_cast<uint8_t>(bf16_to_e4m3(s16[j]));
        return KVT_NO_MOVE;
      }
      const uint32_t done = (len >> 3) << 3;  // stragglers behind the last whole group
      if (threadIdx.x < len - done)
        pk[done + threadIdx.x] = static_cast<uint8_t>(
            bf16_to_e4m3(reinterpret_cast<const uint16_t*>(s8)[done + threadIdx.x]));
    }
    const uint32_t n_groups = len >> 3;  // strided chunks: whole groups by construction
    const uint8_t* src[2];
    bool on[2];
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const uint32_t g = threadIdx.x + (k << 8);
      on[k] = g < n_groups;
      if (it.c.shape == 0) {
        src[k] = cache + 2ull * off + (g << 4);
      } else {
        const StrideShape& s = shapes.shape[it.c.shape - 1u];
        const uint32_t q = (off >> 3) + g;    // group index inside the chunk
        const uint32_t per_rec = s.vlen << 1;  // groups per record
        const uint32_t rec = q / per_rec;
        const uint32_t col = q - rec * per_rec;
        const uint32_t o = s.n_inner == 1 ? rec : (s.n_inner == 2 ? rec >> 1 : rec / s.n_inner);
        const uint32_t i = rec - o * s.n_inner;
        src[k] = cache + o * s.outer[0] + i * s.inner[0] + (col << 4);
      }
    }
    u32x4 in[2];
#pragma unroll
    for (int k = 0; k < 2; ++k) in[k] = load_vec(on[k] ? src[k] : cache);  // both in flight
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      if (!on[k]) continue;
      u32x2 r;
      r.x = cvt4(in[k].x, in[k].y);
      r.y = cvt4(in[k].z, in[k].w);
      uint8_t* d = pk + ((threadIdx.x + (k << 8)) << 3);
      asm volatile("global_store_dwordx2 %0, %1, off sc0 sc1 nt" ::"v"(d), "v"(r) : "memory");
    }
    return KVT_NO_MOVE;
  });
}

// The pipelined capped launch of a converting table (every entry 16-byte aligned on both sides
// and a multiple of 16 elements long): one trip converts V slices of 4096 elements of one
// entry, lane t the groups of 8 elements t, t + 256, ... of the part, each a 16-byte load
// through the cache-side descriptor at an offset computed when the part is fetched, and an
// 8-byte store through the packed-side descriptor. Record arithmetic as in
// strided_entries_kernel, in groups: a record of vlen * 16 elements is 2 * vlen groups.
template <int V>
__device__ __forceinline__ void convert_entries(
    const Chunk* __restrict__ chunks, uint32_t n_chunks, uint32_t part_shift,
    uint8_t* const* __restrict__ layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
    uint32_t n_layers, uint8_t* __restrict__ packed, uint64_t layer_stride, const BlobOffsets& blobs,
    const StrideTable& shapes, uint32_t* tickets) {
  constexpr int G = 2 * V;  // groups per lane and trip
  EntryWalk walk(n_chunks << part_shift, n_layers, tickets, V == 8 ? 3u : (V == 4 ? 2u : 1u));
  const Entry* table = reinterpret_cast<const Entry*>(chunks);
  rsrc_t cdesc[3], pdesc[3];
  u32x4 r[3][G];
  auto next = [&](int k, uint32_t* coff) -> bool {
    uint32_t item, lay;
    bool valid;
    const bool live = walk.next(item, lay, valid);
    const Entry c = table[item >> part_shift];
    const uint32_t begin = (item & ((1u << part_shift) - 1u)) * (static_cast<uint32_t>(V) << kSliceShift);
    uint8_t* cache = layer_ptrs[static_cast<uint64_t>(first_layer + lay) * n_tensors + c.tensor()] + c.cache;
    uint8_t* pk = packed + lay * layer_stride + blobs.off[c.tensor()] + c.packed + begin;
    const uint32_t bytes =
        valid && c.len > begin ? min(c.len - begin, static_cast<uint32_t>(V) << kSliceShift) : 0u;
    pdesc[k] = make_rsrc(pk, bytes);
    cdesc[k] = make_rsrc(cache, bytes ? kCacheWindow : 0u);
    const bool plain = c.shape == 0;
    const u32x16 raw = *reinterpret_cast<const u32x16*>(&shapes.shape[plain ? 0u : c.shape - 1u]);
    const uint32_t vlen = plain ? 0u : raw[0];
    const uint32_t rec_mul = plain || raw[0] == 1u ? 0u : raw[1], rec_add = !plain && raw[0] == 1u ? 1u : 0u;
    const uint32_t n_inner = plain ? 1u : raw[2];
    const uint32_t o_mul = raw[12], o_add = n_inner == 1u ? 1u : 0u;
    const uint32_t outer = raw[4], inner = raw[8];
#pragma unroll
    for (int j = 0; j < G; ++j) {
      const uint32_t g = threadIdx.x + (j << 8);    // group inside the part
      const uint32_t q = (begin >> 3) + g;          // group inside the entry, < 2^16
      const uint32_t half = q >> 1;                 // 16-element vector inside the entry
      const uint32_t rec = __umulhi(half, rec_mul) + half * rec_add;
      const uint32_t col = q - rec * (vlen << 1);
      const uint32_t o = __umulhi(rec, o_mul) + rec * o_add;
      const uint32_t i = rec - o * n_inner;
      coff[j] = (g << 3) < bytes ? o * outer + i * inner + (col << 4) : kNoVector;
    }
    return live;
  };
  // the offsets are used up by the loads that follow at once
  auto fetch = [&](int k) -> bool {
    uint32_t coff[G];
    const bool live = next(k, coff);
#pragma unroll
    for (int j = 0; j < G; ++j)
      r[k][j] = __builtin_amdgcn_raw_buffer_load_b128(cdesc[k], coff[j], 0, kLoadPolicy);
    return live;
  };
  auto nothing = [&](int) {};
  auto store = [&](int k) {
#pragma unroll
    for (int j = 0; j < G; ++j) {
      u32x2 out;
      out.x = cvt4(r[k][j].x, r[k][j].y);
      out.y = cvt4(r[k][j].z, r[k][j].w);
      __builtin_amdgcn_raw_buffer_store_b64(out, pdesc[k], (threadIdx.x + (j << 8)) << 3, 0, kStorePolicy);
    }
  };
  KVT_ROTATE3(fetch, nothing, store);
  walk.leave();
}
template <int V>
__global__ __launch_bounds__(kThreads, 4) void convert_entries_kernel(
    const Chunk* __restrict__ chunks, uint32_t n_chunks, uint32_t part_shift,
    uint8_t* const* __restrict__ layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
    uint32_t n_layers, uint8_t* __restrict__ packed, uint64_t layer_stride, BlobOffsets blobs,
    StrideTable shapes, uint32_t* tickets) {
  convert_entries<V>(chunks, n_chunks, part_shift, layer_ptrs, n_tensors, first_layer, n_layers, packed,
                     layer_stride, blobs, shapes, tickets);
}

// Converting tables with entries of 4096 elements: a wavefront per entry (see
// copy_entries_by_wave_kernel), lane t of the wavefront the groups t, t + 64, ... t + 448.
template <int U>
__device__ __forceinline__ void convert_entries_by_wave(
    const Chunk* __restrict__ chunks, uint32_t n_chunks,
    uint8_t* const* __restrict__ layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
    uint32_t n_layers, uint8_t* __restrict__ packed, uint64_t layer_stride, const BlobOffsets& blobs,
    const StrideTable& shapes, uint32_t* tickets) {
  constexpr int G = 8;  // groups per lane and entry
  EntryWalk walk(n_chunks, n_layers, tickets, 0u);
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t lane = threadIdx.x & 63u;
  const Entry* table = reinterpret_cast<const Entry*>(chunks);
  rsrc_t pdesc[3][U];
  u32x4 r[3][U][G];
  // the cache-side descriptor and the offsets are used up by the loads that follow at once
  auto fetch = [&](int k) -> bool {
    bool live = false;
    uint32_t b[4 * U], l[4 * U];
    bool ok[4 * U];
#pragma unroll
    for (int j = 0; j < 4 * U; ++j) {
      const bool more = walk.next(b[j], l[j], ok[j]);
      if (j == 0) live = more;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      uint32_t item = b[4 * u], lay = l[4 * u];
      bool valid = ok[4 * u];
#pragma unroll
      for (int w = 1; w < 4; ++w)
        if (wave == static_cast<uint32_t>(w)) item = b[4 * u + w], lay = l[4 * u + w], valid = ok[4 * u + w];
      const Entry c = table[item];
      uint8_t* cache = layer_ptrs[static_cast<uint64_t>(first_layer + lay) * n_tensors + c.tensor()] + c.cache;
      uint8_t* pk = packed + lay * layer_stride + blobs.off[c.tensor()] + c.packed;
      const uint32_t bytes = valid ? c.len : 0u;
      pdesc[k][u] = make_rsrc(pk, bytes);
      const rsrc_t cdesc = make_rsrc(cache, bytes ? kCacheWindow : 0u);
      const bool plain = c.shape == 0;
      const u32x16 raw = *reinterpret_cast<const u32x16*>(&shapes.shape[plain ? 0u : c.shape - 1u]);
      const uint32_t vlen = plain ? 0u : raw[0];
      const uint32_t rec_mul = plain || raw[0] == 1u ? 0u : raw[1], rec_add = !plain && raw[0] == 1u ? 1u : 0u;
      const uint32_t n_inner = plain ? 1u : raw[2];
      const uint32_t o_mul = raw[12], o_add = n_inner == 1u ? 1u : 0u;
      const uint32_t outer = raw[4], inner = raw[8];
#pragma unroll
      for (int j = 0; j < G; ++j) {
        const uint32_t q = lane + (j << 6);  // group inside the entry
        const uint32_t half = q >> 1;        // 16-element vector inside the entry
        const uint32_t rec = __umulhi(half, rec_mul) + half * rec_add;
        const uint32_t col = q - rec * (vlen << 1);
        const uint32_t o = __umulhi(rec, o_mul) + rec * o_add;
        const uint32_t i = rec - o * n_inner;
        const uint32_t coff = (q << 3) < bytes ? o * outer + i * inner + (col << 4) : kNoVector;
        r[k][u][j] = __builtin_amdgcn_raw_buffer_load_b128(cdesc, coff, 0, kLoadPolicy);
      }
    }
    return live;
  };
  auto nothing = [&](int) {};
  auto store = [&](int k) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int j = 0; j < G; ++j) {
        u32x2 out;
        out.x = cvt4(r[k][u][j].x, r[k][u][j].y);
        out.y = cvt4(r[k][u][j].z, r[k][u][j].w);
        __builtin_amdgcn_raw_buffer_store_b64(out, pdesc[k][u], (lane + (j << 6)) << 3, 0, kStorePolicy);
      }
  };
  KVT_ROTATE3(fetch, nothing, store);
  walk.leave();
}
template <int U>
__global__ __launch_bounds__(kThreads, 4) void convert_entries_by_wave_kernel(
    const Chunk* __restrict__ chunks, uint32_t n_chunks,
    uint8_t* const* __restrict__ layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
    uint32_t n_layers, uint8_t* __restrict__ packed, uint64_t layer_stride, BlobOffsets blobs,
    StrideTable shapes, uint32_t* tickets) {
  convert_entries_by_wave<U>(chunks, n_chunks, layer_ptrs, n_tensors, first_layer, n_layers, packed,
                             layer_stride, blobs, shapes, tickets);
}

// ------------------------------------------------------------------ plan slots
//
// A slot is a chunk table at a fixed device address whose contents change from batch to batch:
// the launches that read it can be recorded into a hipGraph once and replayed for every batch.
// What varies with the batch -- the number of entries, where each tensor's blob starts in a
// packed layer, the record shapes of strided entries -- lives in a header in front of the table
// and is read here, not passed as kernel arguments; what a recorded launch fixes is the grid,
// so these are the persistent kernels above (whose grid does not depend on the table's length)
// with the header's values in place of the arguments. An empty batch ends every workgroup at once.
#define KVT_SLOT_PARAMS                                                                              \
  const Chunk *__restrict__ chunks, const SlotHeader *__restrict__ hdr,                              \
      uint8_t *const *__restrict__ layer_ptrs, uint32_t n_tensors, uint32_t first_layer,             \
      uint32_t n_layers, uint8_t *packed, uint64_t layer_stride, uint32_t *tickets
#define KVT_SLOT_TAIL layer_ptrs, n_tensors, first_layer, n_layers, packed, layer_stride, hdr->blobs
// A batch so small that no workgroup gets a second trip is dealt out by position: asking for a
// ticket first would put one more round trip to memory in front of the only load (a request of
// 64 entries per layer: 7.2 -> 5.8 us per layer in a replayed graph, of which 3.5 are the launch
// and the signal).
__device__ __forceinline__ uint32_t* slot_tickets(uint32_t n_chunks, uint32_t n_layers, uint32_t per_trip,
                                                  uint32_t* tickets) {
  return static_cast<uint64_t>(n_chunks) * n_layers <= static_cast<uint64_t>(gridDim.x) * per_trip ? nullptr : tickets;
}

template <bool PACK, int V>
__global__ __launch_bounds__(kThreads, 4) void copy_entries_slot_kernel(KVT_SLOT_PARAMS) {
  const uint32_t n_chunks = hdr->n_entries;
  if (n_chunks == 0) return;
  const Entry* table = reinterpret_cast<const Entry*>(chunks);
  copy_entries<PACK, V>([&](uint32_t e) { return table[e]; }, n_chunks, KVT_SLOT_TAIL,
                        slot_tickets(n_chunks, n_layers, 1, tickets));
}
template <bool PACK, int V, int U>
__global__ __launch_bounds__(kThreads, 4) void copy_entries_by_wave_slot_kernel(KVT_SLOT_PARAMS) {
  const uint32_t n_chunks = hdr->n_entries;
  if (n_chunks == 0) return;
  const Entry* table = reinterpret_cast<const Entry*>(chunks);
  copy_entries_by_wave<PACK, V, U>([&](uint32_t e) { return table[e]; }, n_chunks, KVT_SLOT_TAIL,
                                   slot_tickets(n_chunks, n_layers, 4 * U, tickets));
}
template <bool PACK, int V>
__global__ __launch_bounds__(kThreads, 4) void strided_entries_slot_kernel(KVT_SLOT_PARAMS, uint32_t part_shift) {
  const uint32_t n_chunks = hdr->n_entries;
  if (n_chunks == 0) return;
  const uint32_t lane = threadIdx.x << 4;
  entries_pipeline<PACK, V>(chunks, n_chunks, part_shift, KVT_SLOT_TAIL,
                            slot_tickets(n_chunks << part_shift, n_layers, 1, tickets),
                            [&](const Entry& c, uint32_t begin, uint32_t bytes, uint32_t* coff) {
                              strided_offsets<PACK, V, kSliceShift>(hdr->shapes, c, begin, bytes, lane, coff);
                            });
}
template <bool PACK, int V, int U>
__global__ __launch_bounds__(kThreads, 4) void strided_entries_by_wave_slot_kernel(KVT_SLOT_PARAMS) {
  const uint32_t n_chunks = hdr->n_entries;
  if (n_chunks == 0) return;
  const uint32_t lane = (threadIdx.x & 63u) << 4;
  entries_pipeline_by_wave<PACK, V, U>(chunks, n_chunks, KVT_SLOT_TAIL, slot_tickets(n_chunks, n_layers, 4 * U, tickets),
                                       [&](const Entry& c, uint32_t bytes, uint32_t* coff) {
                                         strided_offsets<PACK, V, 10>(hdr->shapes, c, 0u, bytes, lane, coff);
                                       });
}
template <bool PACK, int V>
__global__ __launch_bounds__(kThreads, 4) void xform_entries_slot_kernel(KVT_SLOT_PARAMS, uint32_t part_shift,
                                                                        XformDev x) {
  const uint32_t n_chunks = hdr->n_entries;
  if (n_chunks == 0) return;
  const uint32_t lane = threadIdx.x << 4;
  entries_pipeline<PACK, V>(chunks, n_chunks, part_shift, KVT_SLOT_TAIL,
                            slot_tickets(n_chunks << part_shift, n_layers, 1, tickets),
                            [&](const Entry& c, uint32_t begin, uint32_t bytes, uint32_t* coff) {
                              xform_offsets<V, kSliceShift>(x, c, begin, bytes, lane, coff);
                            });
}
template <bool PACK, int V, int U>
__global__ __launch_bounds__(kThreads, 4) void xform_entries_by_wave_slot_kernel(KVT_SLOT_PARAMS, XformDev x) {
  const uint32_t n_chunks = hdr->n_entries;
  if (n_chunks == 0) return;
  const uint32_t lane = (threadIdx.x & 63u) << 4;
  entries_pipeline_by_wave<PACK, V, U>(chunks, n_chunks, KVT_SLOT_TAIL, slot_tickets(n_chunks, n_layers, 4 * U, tickets),
                                       [&](const Entry& c, uint32_t bytes, uint32_t* coff) {
                                         xform_offsets<V, 10>(x, c, 0u, bytes, lane, coff);
                                       });
}
template <int V>
__global__ __launch_bounds__(kThreads, 4) void convert_entries_slot_kernel(KVT_SLOT_PARAMS, uint32_t part_shift) {
  const uint32_t n_chunks = hdr->n_entries;
  if (n_chunks == 0) return;
  convert_entries<V>(chunks, n_chunks, part_shift, KVT_SLOT_TAIL, hdr->shapes,
                     slot_tickets(n_chunks << part_shift, n_layers, 1, tickets));
}
__global__ __launch_bounds__(kThreads, 4) void convert_entries_by_wave_slot_kernel(KVT_SLOT_PARAMS) {
  const uint32_t n_chunks = hdr->n_entries;
  if (n_chunks == 0) return;
  convert_entries_by_wave<1>(chunks, n_chunks, KVT_SLOT_TAIL, hdr->shapes, slot_tickets(n_chunks, n_layers, 4, tickets));
}

// Plain linear copy with the gather kernel's slice shape (calibration / ceiling).
__global__ __launch_bounds__(kThreads) void copy_linear_kernel(uint8_t* __restrict__ dst,
                                                               const uint8_t* __restrict__ src,
                                                               uint64_t bytes, uint32_t n_slices) {
  const uint32_t b = xcd_remap(blockIdx.x, n_slices);
  if (b >= n_slices) return;
  const uint64_t begin = static_cast<uint64_t>(b) << kSliceShift;
  const uint64_t m = bytes - begin;
  copy_slice(dst + begin, src + begin, static_cast<uint32_t>(m < kSlice ? m : kSlice), threadIdx.x);
}

// ----------------------------------------------------------------- launchers

static uint32_t round8(uint32_t n) { return (n + 7u) & ~7u; }

// Grid of a chunk launch: one workgroup per (slice, layer); or, when the caller limits the
// launch to max_wgs workgroups and there are more items than that, max_wgs workgroups
// (rounded down to a multiple of 8, at least 8) that stride over the items.
struct ChunkGrid {
  dim3 grid;
  bool capped;
};
static ChunkGrid chunk_grid(uint32_t n_slices, uint32_t n_layers, uint32_t max_wgs) {
  const uint32_t per_layer = round8(n_slices);
  const uint32_t cap = max_wgs < 8u ? 8u : (max_wgs & ~7u);
  if (max_wgs == 0 || static_cast<uint64_t>(per_layer) * n_layers <= cap)
    return ChunkGrid{dim3(per_layer, n_layers), false};
  return ChunkGrid{dim3(cap), true};
}

#define KVT_LAUNCH_CHUNKS(KERNEL, ...)                                                          \
  hipLaunchKernelGGL(KERNEL, g.grid, dim3(kThreads), 0, stream, __VA_ARGS__)

hipError_t launch_copy_chunks(bool pack, const Chunk* chunks, uint32_t n_chunks,
                              uint32_t sub_shift, uint8_t* const* layer_ptrs, uint32_t n_tensors,
                              uint32_t first_layer, uint32_t n_layers, uint8_t* packed,
                              uint64_t layer_stride, const BlobOffsets& blobs, uint32_t max_wgs, bool pipelined,
                              uint32_t policy, uint32_t* tickets, hipStream_t stream) {
  if (n_chunks == 0 || n_layers == 0) return hipSuccess;
  const uint32_t n_slices = n_chunks << sub_shift;
  const ChunkGrid g = chunk_grid(n_slices, n_layers, max_wgs);
  if (!g.capped) tickets = nullptr;
  const uint32_t shift_arg = sub_shift | (g.capped ? 0u : (policy & 3u) << 8);
#define KVT_ARGS chunks, n_slices, shift_arg, layer_ptrs, n_tensors, first_layer, n_layers, packed, layer_stride, blobs, tickets
  if (!g.capped) {
    if (pack) KVT_LAUNCH_CHUNKS((copy_chunks_kernel<true, kOnePerSlice>), KVT_ARGS);
    else KVT_LAUNCH_CHUNKS((copy_chunks_kernel<false, kOnePerSlice>), KVT_ARGS);
  } else if (!pipelined) {
    if (pack) KVT_LAUNCH_CHUNKS((copy_chunks_kernel<true, kStriding>), KVT_ARGS);
    else KVT_LAUNCH_CHUNKS((copy_chunks_kernel<false, kStriding>), KVT_ARGS);
  } else {
    if (pack) KVT_LAUNCH_CHUNKS((copy_chunks_kernel<true, kPipelined>), KVT_ARGS);
    else KVT_LAUNCH_CHUNKS((copy_chunks_kernel<false, kPipelined>), KVT_ARGS);
  }
#undef KVT_ARGS
  return hipGetLastError();
}

// One entry per workgroup and trip (entries of 16 or 32 KiB), or per wavefront (4 or 8 KiB: two
// entries of 4 KiB or one of 8 KiB per wavefront and trip; more per trip, or five register
// sets, were slower from one workgroup per CU on).
#define KVT_LAUNCH_ENTRIES(LARGE, BY_WAVE, TABLE)                                                   \
  do {                                                                                              \
    const dim3 grid(wgs), block(kThreads);                                                          \
    switch ((sub_shift << 1) | (pack ? 1u : 0u)) {                                                  \
      case 0: hipLaunchKernelGGL((BY_WAVE<false, 4, 2>), grid, block, 0, stream, TABLE, KVT_ENTRIES_ARGS); break; \
      case 1: hipLaunchKernelGGL((BY_WAVE<true, 4, 2>), grid, block, 0, stream, TABLE, KVT_ENTRIES_ARGS); break;  \
      case 2: hipLaunchKernelGGL((BY_WAVE<false, 8, 1>), grid, block, 0, stream, TABLE, KVT_ENTRIES_ARGS); break; \
      case 3: hipLaunchKernelGGL((BY_WAVE<true, 8, 1>), grid, block, 0, stream, TABLE, KVT_ENTRIES_ARGS); break;  \
      case 4: hipLaunchKernelGGL((LARGE<false, 4>), grid, block, 0, stream, TABLE, KVT_ENTRIES_ARGS); break;      \
      case 5: hipLaunchKernelGGL((LARGE<true, 4>), grid, block, 0, stream, TABLE, KVT_ENTRIES_ARGS); break;       \
      case 6: hipLaunchKernelGGL((LARGE<false, 8>), grid, block, 0, stream, TABLE, KVT_ENTRIES_ARGS); break;      \
      default: hipLaunchKernelGGL((LARGE<true, 8>), grid, block, 0, stream, TABLE, KVT_ENTRIES_ARGS); break;      \
    }                                                                                               \
  } while (0)

hipError_t launch_copy_entries(bool pack, const Chunk* chunks, uint32_t n_chunks, uint32_t sub_shift,
                               uint8_t* const* layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
                               uint32_t n_layers, uint8_t* packed, uint64_t layer_stride,
                               const BlobOffsets& blobs, uint32_t wgs, uint32_t* tickets, hipStream_t stream) {
  if (n_chunks == 0 || n_layers == 0) return hipSuccess;
  if (sub_shift > 3 || wgs < 8 || (wgs & 7u)) return hipErrorInvalidValue;
  KVT_LAUNCH_ENTRIES(copy_entries_kernel, copy_entries_by_wave_kernel, chunks);
  return hipGetLastError();
}

hipError_t launch_copy_entries_small(bool pack, const SmallTable& table, uint32_t n_chunks,
                                     uint32_t sub_shift, uint8_t* const* layer_ptrs, uint32_t n_tensors,
                                     uint32_t first_layer, uint32_t n_layers, uint8_t* packed,
                                     uint64_t layer_stride, const BlobOffsets& blobs, uint32_t wgs,
                                     hipStream_t stream) {
  if (n_chunks == 0 || n_layers == 0) return hipSuccess;
  if (sub_shift > 3 || wgs < 8 || (wgs & 7u)) return hipErrorInvalidValue;
  uint32_t* const tickets = nullptr;  // a short table's launch is over before their order pays
  KVT_LAUNCH_ENTRIES(copy_entries_small_kernel, copy_entries_by_wave_small_kernel, table);
  return hipGetLastError();
}
#undef KVT_LAUNCH_ENTRIES

// V slices per trip and the parts an entry is taken in, for entries of 4096 << sub_shift bytes.
static bool entries_shape(uint32_t sub_shift, uint32_t wgs, int max_v, int* v, uint32_t* part_shift) {
  if (sub_shift < 1 || sub_shift > 7 || wgs < 8 || (wgs & 7u)) return false;
  *v = sub_shift == 1 ? 2 : (sub_shift == 2 ? 4 : max_v);
  *part_shift = sub_shift - (*v == 2 ? 1u : (*v == 4 ? 2u : 3u));
  return true;
}

hipError_t launch_strided_entries(bool pack, const Chunk* chunks, uint32_t n_chunks, uint32_t sub_shift,
                                  uint8_t* const* layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
                                  uint32_t n_layers, uint8_t* packed, uint64_t layer_stride,
                                  const BlobOffsets& blobs, const StrideTable& shapes, uint32_t wgs,
                                  uint32_t* tickets, hipStream_t stream) {
  if (n_chunks == 0 || n_layers == 0) return hipSuccess;
  int v = 0;
  uint32_t part_shift = 0;
  if (!entries_shape(sub_shift, wgs, 8, &v, &part_shift)) return hipErrorInvalidValue;
  const dim3 grid(wgs), block(kThreads);
#define KVT_ARGS chunks, n_chunks, part_shift, layer_ptrs, n_tensors, first_layer, n_layers, packed, layer_stride, blobs, shapes, tickets
  if (v == 8) {
    if (pack) hipLaunchKernelGGL((strided_entries_kernel<true, 8>), grid, block, 0, stream, KVT_ARGS);
    else hipLaunchKernelGGL((strided_entries_kernel<false, 8>), grid, block, 0, stream, KVT_ARGS);
  } else if (v == 4) {
    if (pack) hipLaunchKernelGGL((strided_entries_kernel<true, 4>), grid, block, 0, stream, KVT_ARGS);
    else hipLaunchKernelGGL((strided_entries_kernel<false, 4>), grid, block, 0, stream, KVT_ARGS);
  } else {
    return hipErrorInvalidValue;  // entries of 4 or 8 KiB: launch_strided_entries_by_wave
  }
#undef KVT_ARGS
  return hipGetLastError();
}

hipError_t launch_strided_entries_by_wave(bool pack, const Chunk* chunks, uint32_t n_chunks, uint32_t sub_shift,
                                          uint8_t* const* layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
                                          uint32_t n_layers, uint8_t* packed, uint64_t layer_stride,
                                          const BlobOffsets& blobs, const StrideTable& shapes, uint32_t wgs,
                                          uint32_t* tickets, hipStream_t stream) {
  if (n_chunks == 0 || n_layers == 0) return hipSuccess;
  if (sub_shift > 1 || wgs < 8 || (wgs & 7u)) return hipErrorInvalidValue;
  const dim3 grid(wgs), block(kThreads);
#define KVT_ARGS chunks, n_chunks, layer_ptrs, n_tensors, first_layer, n_layers, packed, layer_stride, blobs, shapes, tickets
  if (sub_shift == 0) {
    if (pack) hipLaunchKernelGGL((strided_entries_by_wave_kernel<true, 4, 2>), grid, block, 0, stream, KVT_ARGS);
    else hipLaunchKernelGGL((strided_entries_by_wave_kernel<false, 4, 2>), grid, block, 0, stream, KVT_ARGS);
  } else {
    if (pack) hipLaunchKernelGGL((strided_entries_by_wave_kernel<true, 8, 1>), grid, block, 0, stream, KVT_ARGS);
    else hipLaunchKernelGGL((strided_entries_by_wave_kernel<false, 8, 1>), grid, block, 0, stream, KVT_ARGS);
  }
#undef KVT_ARGS
  return hipGetLastError();
}

hipError_t launch_convert_entries(const Chunk* chunks, uint32_t n_chunks, uint32_t sub_shift,
                                  uint8_t* const* layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
                                  uint32_t n_layers, uint8_t* packed, uint64_t layer_stride,
                                  const BlobOffsets& blobs, const StrideTable& shapes, uint32_t wgs,
                                  uint32_t* tickets, hipStream_t stream) {
  if (n_chunks == 0 || n_layers == 0) return hipSuccess;
  const dim3 grid(wgs), block(kThreads);
  if (sub_shift == 0) {  // entries of 4096 elements: a wavefront each
    if (wgs < 8 || (wgs & 7u)) return hipErrorInvalidValue;
    hipLaunchKernelGGL((convert_entries_by_wave_kernel<1>), grid, block, 0, stream, chunks, n_chunks, layer_ptrs,
                       n_tensors, first_layer, n_layers, packed, layer_stride, blobs, shapes, tickets);
    return hipGetLastError();
  }
  int v = 0;
  uint32_t part_shift = 0;
  if (!entries_shape(sub_shift, wgs, 4, &v, &part_shift)) return hipErrorInvalidValue;
#define KVT_ARGS chunks, n_chunks, part_shift, layer_ptrs, n_tensors, first_layer, n_layers, packed, layer_stride, blobs, shapes, tickets
  if (v == 4) hipLaunchKernelGGL((convert_entries_kernel<4>), grid, block, 0, stream, KVT_ARGS);
  else hipLaunchKernelGGL((convert_entries_kernel<2>), grid, block, 0, stream, KVT_ARGS);
#undef KVT_ARGS
  return hipGetLastError();
}

hipError_t launch_xform_entries(bool pack, const Chunk* chunks, uint32_t n_chunks, uint32_t sub_shift,
                                uint8_t* const* layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
                                uint32_t n_layers, uint8_t* packed, uint64_t layer_stride,
                                const BlobOffsets& blobs, const XformDev& x, uint32_t wgs,
                                uint32_t* tickets, hipStream_t stream) {
  if (n_chunks == 0 || n_layers == 0) return hipSuccess;
  int v = 0;
  uint32_t part_shift = 0;
  const dim3 grid(wgs), block(kThreads);
  if (sub_shift <= 1) {  // half pages of 4 or 8 KiB: a wavefront per entry
    if (wgs < 8 || (wgs & 7u)) return hipErrorInvalidValue;
#define KVT_ARGS chunks, n_chunks, layer_ptrs, n_tensors, first_layer, n_layers, packed, layer_stride, blobs, x, tickets
    if (sub_shift == 0) {
      if (pack) hipLaunchKernelGGL((xform_entries_by_wave_kernel<true, 4, 2>), grid, block, 0, stream, KVT_ARGS);
      else hipLaunchKernelGGL((xform_entries_by_wave_kernel<false, 4, 2>), grid, block, 0, stream, KVT_ARGS);
    } else {
      if (pack) hipLaunchKernelGGL((xform_entries_by_wave_kernel<true, 8, 1>), grid, block, 0, stream, KVT_ARGS);
      else hipLaunchKernelGGL((xform_entries_by_wave_kernel<false, 8, 1>), grid, block, 0, stream, KVT_ARGS);
    }
#undef KVT_ARGS
    return hipGetLastError();
  }
  // the scatter keeps its offsets until the stores: 8 slices per trip would not fit the registers
  if (!entries_shape(sub_shift, wgs, pack ? 8 : 4, &v, &part_shift)) return hipErrorInvalidValue;
#define KVT_ARGS chunks, n_chunks, part_shift, layer_ptrs, n_tensors, first_layer, n_layers, packed, layer_stride, blobs, x, tickets
  if (v == 8) {
    hipLaunchKernelGGL((xform_entries_kernel<true, 8>), grid, block, 0, stream, KVT_ARGS);
  } else {
    if (pack) hipLaunchKernelGGL((xform_entries_kernel<true, 4>), grid, block, 0, stream, KVT_ARGS);
    else hipLaunchKernelGGL((xform_entries_kernel<false, 4>), grid, block, 0, stream, KVT_ARGS);
  }
#undef KVT_ARGS
  return hipGetLastError();
}

hipError_t launch_copy_chunks_small(bool pack, const SmallTable& table, uint32_t n_chunks,
                                    uint32_t sub_shift, uint8_t* const* layer_ptrs,
                                    uint32_t n_tensors, uint32_t first_layer, uint32_t n_layers,
                                    uint8_t* packed, uint64_t layer_stride,
                                    const BlobOffsets& blobs, uint32_t max_wgs, bool pipelined,
                                    uint32_t policy, uint32_t* tickets, hipStream_t stream) {
  if (n_chunks == 0 || n_layers == 0) return hipSuccess;
  const uint32_t n_slices = n_chunks << sub_shift;
  const ChunkGrid g = chunk_grid(n_slices, n_layers, max_wgs);
  if (!g.capped) tickets = nullptr;
  const uint32_t shift_arg = sub_shift | (g.capped ? 0u : (policy & 3u) << 8);
#define KVT_ARGS table, n_slices, shift_arg, layer_ptrs, n_tensors, first_layer, n_layers, packed, layer_stride, blobs, tickets
  if (!g.capped) {
    if (pack) KVT_LAUNCH_CHUNKS((copy_chunks_small_kernel<true, kOnePerSlice>), KVT_ARGS);
    else KVT_LAUNCH_CHUNKS((copy_chunks_small_kernel<false, kOnePerSlice>), KVT_ARGS);
  } else if (!pipelined) {
    if (pack) KVT_LAUNCH_CHUNKS((copy_chunks_small_kernel<true, kStriding>), KVT_ARGS);
    else KVT_LAUNCH_CHUNKS((copy_chunks_small_kernel<false, kStriding>), KVT_ARGS);
  } else {
    if (pack) KVT_LAUNCH_CHUNKS((copy_chunks_small_kernel<true, kPipelined>), KVT_ARGS);
    else KVT_LAUNCH_CHUNKS((copy_chunks_small_kernel<false, kPipelined>), KVT_ARGS);
  }
#undef KVT_ARGS
  return hipGetLastError();
}

hipError_t launch_strided_chunks(bool pack, const Chunk* chunks, uint32_t n_chunks,
                                 uint32_t sub_shift, uint8_t* const* layer_ptrs,
                                 uint32_t n_tensors, uint32_t first_layer, uint32_t n_layers,
                                 uint8_t* packed, uint64_t layer_stride, const BlobOffsets& blobs,
                                 const StrideTable& shapes, bool words, uint32_t max_wgs, uint32_t policy,
                                 uint32_t* tickets, hipStream_t stream) {
  if (n_chunks == 0 || n_layers == 0) return hipSuccess;
  const uint32_t n_slices = n_chunks << sub_shift;
  const ChunkGrid g = chunk_grid(n_slices, n_layers, max_wgs);
  if (!g.capped) tickets = nullptr;
  const uint32_t shift_arg = sub_shift | (g.capped ? 0u : (policy & 3u) << 8);
#define KVT_ARGS chunks, n_slices, shift_arg, layer_ptrs, n_tensors, first_layer, n_layers, packed, layer_stride, blobs, shapes, tickets
#define KVT_STRIDED(P, W)                                                                       \
  do {                                                                                          \
    if (g.capped) KVT_LAUNCH_CHUNKS((strided_chunks_kernel<P, W, true>), KVT_ARGS);             \
    else KVT_LAUNCH_CHUNKS((strided_chunks_kernel<P, W, false>), KVT_ARGS);                     \
  } while (0)
  if (pack && !words) KVT_STRIDED(true, false);
  else if (pack) KVT_STRIDED(true, true);
  else if (!words) KVT_STRIDED(false, false);
  else KVT_STRIDED(false, true);
#undef KVT_STRIDED
#undef KVT_ARGS
  return hipGetLastError();
}

hipError_t launch_convert_chunks(const Chunk* chunks, uint32_t n_chunks, uint32_t sub_shift,
                                 uint8_t* const* layer_ptrs, uint32_t n_tensors,
                                 uint32_t first_layer, uint32_t n_layers, uint8_t* packed,
                                 uint64_t layer_stride, const BlobOffsets& blobs,
                                 const StrideTable& shapes, uint32_t max_wgs, uint32_t* tickets,
                                 hipStream_t stream) {
  if (n_chunks == 0 || n_layers == 0) return hipSuccess;
  const uint32_t n_slices = n_chunks << sub_shift;
  const ChunkGrid g = chunk_grid(n_slices, n_layers, max_wgs);
  if (!g.capped) tickets = nullptr;
#define KVT_ARGS chunks, n_slices, sub_shift, layer_ptrs, n_tensors, first_layer, n_layers, packed, layer_stride, blobs, shapes, tickets
  if (g.capped) KVT_LAUNCH_CHUNKS((convert_chunks_kernel<true>), KVT_ARGS);
  else KVT_LAUNCH_CHUNKS((convert_chunks_kernel<false>), KVT_ARGS);
#undef KVT_ARGS
  return hipGetLastError();
}

hipError_t launch_xform_chunks(bool pack, const Chunk* chunks, uint32_t n_chunks,
                               uint32_t sub_shift, uint8_t* const* layer_ptrs, uint32_t n_tensors,
                               uint32_t first_layer, uint32_t n_layers, uint8_t* packed,
                               uint64_t layer_stride, const BlobOffsets& blobs, const XformDev& x,
                               uint32_t max_wgs, uint32_t policy, uint32_t* tickets, hipStream_t stream) {
  if (n_chunks == 0 || n_layers == 0) return hipSuccess;
  const uint32_t n_slices = n_chunks << sub_shift;
  const ChunkGrid g = chunk_grid(n_slices, n_layers, max_wgs);
  if (!g.capped) tickets = nullptr;
  const uint32_t shift_arg = sub_shift | (g.capped ? 0u : (policy & 3u) << 8);
#define KVT_ARGS chunks, n_slices, shift_arg, layer_ptrs, n_tensors, first_layer, n_layers, packed, layer_stride, blobs, x, tickets
  if (pack && !g.capped) KVT_LAUNCH_CHUNKS((xform_chunks_kernel<true, false>), KVT_ARGS);
  else if (pack) KVT_LAUNCH_CHUNKS((xform_chunks_kernel<true, true>), KVT_ARGS);
  else if (!g.capped) KVT_LAUNCH_CHUNKS((xform_chunks_kernel<false, false>), KVT_ARGS);
  else KVT_LAUNCH_CHUNKS((xform_chunks_kernel<false, true>), KVT_ARGS);
#undef KVT_ARGS
  return hipGetLastError();
}
#undef KVT_LAUNCH_CHUNKS

// grid.y is limited to 65535; the kernels stride over the ranges anyway. max_wgs > 0 limits
// the whole grid (rows x ranges) to that many workgroups.
static dim3 range_grid(int num_wg, int rows, uint32_t max_wgs) {
  uint32_t gx = rows < 1 ? 1u : static_cast<uint32_t>(rows);
  uint32_t gy = num_wg < 65535 ? (num_wg < 1 ? 1u : static_cast<uint32_t>(num_wg)) : 65535u;
  if (max_wgs) {
    if (gx > max_wgs) gx = max_wgs;
    if (gy > max_wgs / gx) gy = max_wgs / gx;
  }
  return dim3(gx, gy);
}

hipError_t launch_copy_ranges_persistent(bool convert, const void* src_base, void* dst_base,
                                         const int64_t* src_off, const int64_t* dst_off,
                                         const int64_t* lens, int64_t n, uint32_t wgs, int walkers,
                                         uint32_t* share, hipStream_t stream) {
  if (n <= 0) return hipSuccess;
  if (n > 0x7FFFFFF0ll || wgs < 8 || (wgs & 7u)) return hipErrorInvalidValue;
  if (convert) share = nullptr;
#define KVT_RANGES(U)                                                                              \
  hipLaunchKernelGGL(copy_ranges_persistent_kernel<U>, dim3(wgs), dim3(kThreads), 0, stream,       \
                     static_cast<const uint8_t*>(src_base), static_cast<uint8_t*>(dst_base), src_off, \
                     dst_off, lens, static_cast<uint32_t>(n), share)
  if (convert)
    hipLaunchKernelGGL(convert_ranges_persistent_kernel, dim3(wgs), dim3(kThreads), 0, stream,
                       static_cast<const uint8_t*>(src_base), static_cast<uint8_t*>(dst_base), src_off,
                       dst_off, lens, static_cast<uint32_t>(n));
  else if (walkers >= 4)
    KVT_RANGES(4);
  else if (walkers >= 2)
    KVT_RANGES(2);
  else
    KVT_RANGES(1);
#undef KVT_RANGES
  if (share)
    hipLaunchKernelGGL(move_listed_ranges_kernel, dim3(wgs), dim3(kThreads), 0, stream,
                       static_cast<const uint8_t*>(src_base), static_cast<uint8_t*>(dst_base), src_off,
                       dst_off, lens, share);
  return hipGetLastError();
}

hipError_t launch_copy_ranges(const void* src_base, void* dst_base, const int64_t* src_off,
                              const int64_t* dst_off, const int64_t* lens, int64_t n, int num_wg,
                              int rows, uint32_t max_wgs, hipStream_t stream) {
  if (n <= 0) return hipSuccess;
  hipLaunchKernelGGL(copy_ranges_kernel, range_grid(num_wg, rows, max_wgs), dim3(kThreads), 0,
                     stream, static_cast<const uint8_t*>(src_base),
                     static_cast<uint8_t*>(dst_base), src_off, dst_off, lens, n);
  return hipGetLastError();
}

hipError_t launch_convert_ranges(const void* src_base, void* dst_base, const int64_t* src_off,
                                 const int64_t* dst_off, const int64_t* lens, int64_t n,
                                 int num_wg, int rows, uint32_t max_wgs, hipStream_t stream) {
  if (n <= 0) return hipSuccess;
  hipLaunchKernelGGL(convert_ranges_kernel, range_grid(num_wg, rows, max_wgs), dim3(kThreads), 0,
                     stream, static_cast<const uint8_t*>(src_base),
                     static_cast<uint8_t*>(dst_base), src_off, dst_off, lens, n);
  return hipGetLastError();
}

hipError_t launch_slot(int kind, bool pack, const Chunk* chunks, const SlotHeader* hdr, uint32_t sub_shift,
                       uint8_t* const* layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
                       uint32_t n_layers, uint8_t* packed, uint64_t layer_stride, const XformDev& x,
                       uint32_t wgs, uint32_t* tickets, hipStream_t stream) {
  if (n_layers == 0) return hipSuccess;
  if (wgs < 8 || (wgs & 7u) || sub_shift > 7) return hipErrorInvalidValue;
  const dim3 grid(wgs), block(kThreads);
#define KVT_ARGS chunks, hdr, layer_ptrs, n_tensors, first_layer, n_layers, packed, layer_stride, tickets
#define KVT_GO(KERNEL, ...) hipLaunchKernelGGL(KERNEL, grid, block, 0, stream, KVT_ARGS, ##__VA_ARGS__)
#define KVT_EITHER(KERNEL_PACK, KERNEL_UNPACK, ...) \
  do {                                              \
    if (pack) KVT_GO(KERNEL_PACK, ##__VA_ARGS__);   \
    else KVT_GO(KERNEL_UNPACK, ##__VA_ARGS__);      \
  } while (0)
  int v = 0;
  uint32_t part_shift = 0;
  if (kind == kSlotPlain || (kind == kSlotConvert && !pack)) {
    // (the unpack of a converting table moves plain fp8 bytes, but its entries may be strided)
    if (kind == kSlotConvert) goto strided;
    if (sub_shift > 3) return hipErrorInvalidValue;
    switch (sub_shift) {
      case 0: KVT_EITHER((copy_entries_by_wave_slot_kernel<true, 4, 2>), (copy_entries_by_wave_slot_kernel<false, 4, 2>)); break;
      case 1: KVT_EITHER((copy_entries_by_wave_slot_kernel<true, 8, 1>), (copy_entries_by_wave_slot_kernel<false, 8, 1>)); break;
      case 2: KVT_EITHER((copy_entries_slot_kernel<true, 4>), (copy_entries_slot_kernel<false, 4>)); break;
      default: KVT_EITHER((copy_entries_slot_kernel<true, 8>), (copy_entries_slot_kernel<false, 8>)); break;
    }
    return hipGetLastError();
  }
  if (kind == kSlotXform) {
    if (sub_shift == 0) {
      KVT_EITHER((xform_entries_by_wave_slot_kernel<true, 4, 2>), (xform_entries_by_wave_slot_kernel<false, 4, 2>), x);
    } else if (sub_shift == 1) {
      KVT_EITHER((xform_entries_by_wave_slot_kernel<true, 8, 1>), (xform_entries_by_wave_slot_kernel<false, 8, 1>), x);
    } else {
      // the scatter keeps its offsets until the stores: 8 slices per trip would not fit the registers
      if (!entries_shape(sub_shift, wgs, pack ? 8 : 4, &v, &part_shift)) return hipErrorInvalidValue;
      if (v == 8) KVT_GO((xform_entries_slot_kernel<true, 8>), part_shift, x);
      else KVT_EITHER((xform_entries_slot_kernel<true, 4>), (xform_entries_slot_kernel<false, 4>), part_shift, x);
    }
    return hipGetLastError();
  }
  if (kind == kSlotConvert) {
    if (sub_shift == 0) {
      KVT_GO(convert_entries_by_wave_slot_kernel);
    } else {
      if (!entries_shape(sub_shift, wgs, 4, &v, &part_shift)) return hipErrorInvalidValue;
      if (v == 4) KVT_GO((convert_entries_slot_kernel<4>), part_shift);
      else KVT_GO((convert_entries_slot_kernel<2>), part_shift);
    }
    return hipGetLastError();
  }
strided:
  if (sub_shift == 0) {
    KVT_EITHER((strided_entries_by_wave_slot_kernel<true, 4, 2>), (strided_entries_by_wave_slot_kernel<false, 4, 2>));
  } else if (sub_shift == 1) {
    KVT_EITHER((strided_entries_by_wave_slot_kernel<true, 8, 1>), (strided_entries_by_wave_slot_kernel<false, 8, 1>));
  } else {
    if (!entries_shape(sub_shift, wgs, 8, &v, &part_shift)) return hipErrorInvalidValue;
    if (v == 8) KVT_EITHER((strided_entries_slot_kernel<true, 8>), (strided_entries_slot_kernel<false, 8>), part_shift);
    else KVT_EITHER((strided_entries_slot_kernel<true, 4>), (strided_entries_slot_kernel<false, 4>), part_shift);
  }
  return hipGetLastError();
#undef KVT_EITHER
#undef KVT_GO
#undef KVT_ARGS
}

hipError_t launch_copy_linear(void* dst, const void* src, uint64_t bytes, hipStream_t stream) {
  if (bytes == 0) return hipSuccess;
  const uint32_t n_slices = static_cast<uint32_t>((bytes + kSlice - 1) >> kSliceShift);
  hipLaunchKernelGGL(copy_linear_kernel, dim3(round8(n_slices)), dim3(kThreads), 0, stream,
                     static_cast<uint8_t*>(dst), static_cast<const uint8_t*>(src), bytes, n_slices);
  return hipGetLastError();
}

}  // namespace kvt
