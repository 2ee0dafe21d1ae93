// Types and launcher declarations shared between the HIP translation units.
#ifndef KVT_DEVICE_H_
#define KVT_DEVICE_H_

#include <hip/hip_runtime.h>

#include <cstdint>

namespace kvt {

// One bounded piece of a range, resident in device memory. 32 bytes. The pack
// and the unpack direction each have their own table (sorted by their cache
// side), so an entry carries a single cache offset.
struct __attribute__((aligned(16))) Chunk {
  uint64_t cache;      // byte offset in the layer tensor (source for pack, destination for unpack)
  uint64_t packed;     // byte offset inside the tensor's blob of one packed layer
  uint32_t len;        // bytes, <= 4096 << sub_shift of the plan
  uint16_t tensor;     // cache tensor index within the layer
  uint16_t t0;         // layout transform only: first token of the half page covered
  uint32_t shape;      // strided plans only: 1 + index into the StrideTable, 0 = contiguous
  uint32_t reserved;
};
static_assert(sizeof(Chunk) == 32, "Chunk must stay 32 bytes");

// Where each cache tensor's blob starts inside one packed layer (kernel argument).
struct BlobOffsets {
  uint64_t off[8];
};

// Device-side constants of the HND <-> NHD page transform.
struct XformDev {
  uint32_t heads, ntpb, vrow;     // vrow = 16-byte vectors per (token, head) row
  uint32_t inv_vrow, inv_heads;   // floor(2^32 / d) + 1: exact quotients for operands < 2^16
};

// Record shape of a strided chunk: the packed side is a dense sequence of
// records of vlen 16-byte vectors; record r lives in the cache at
//   chunk.cache + (r / n_inner) * outer + (r % n_inner) * inner
// (per token: the outer step; K and V of one token: the inner step).
struct __attribute__((aligned(16))) StrideShape {
  uint32_t vlen, inv_vlen;     // inv_vlen = floor(2^32 / vlen) + 1, exact for operands < 2^32 / vlen
  uint32_t n_inner;
  uint32_t inv_wlen;           // the same reciprocal for the record length in 4-byte words (4 * vlen)
  uint64_t outer[2], inner[2];  // [0] = source side (pack), [1] = destination side (unpack)
  uint32_t inv_inner;          // floor(2^32 / n_inner) + 1 (n_inner > 1: exact for operands < 2^16), else 0
  uint32_t reserved[3];
};
static_assert(sizeof(StrideShape) == 64, "StrideShape is read as one 64-byte scalar load");
constexpr uint32_t kMaxShapes = 16;
enum : uint32_t { kPolicyTemporalLoads = 1u, kPolicyCachedStores = 2u };
// Default payload (bytes moved one way) up to which a launch reads with plain loads: none.
// Plain loads pay only when the same data is read again soon (kvt_set_copy_cached_load_max).
constexpr uint64_t kTemporalMaxBytes = 0;
struct StrideTable {
  StrideShape shape[kMaxShapes];
};

// What stands in front of a slot's table in device memory (a plan slot: a table at a fixed
// address that is refilled for every batch, so that launches recorded into a hipGraph find the
// new batch on every replay): everything a launch would otherwise get as an argument and that
// changes with the batch.
struct __attribute__((aligned(256))) SlotHeader {
  uint32_t n_entries;       // table entries of the batch in the slot (0: nothing to move)
  uint32_t reserved[3];
  BlobOffsets blobs;
  uint8_t pad[256 - 16 - sizeof(BlobOffsets)];
  StrideTable shapes;       // record shapes of strided entries (slots made for runs)
};
static_assert(sizeof(SlotHeader) == 256 + sizeof(StrideTable), "SlotHeader layout");
constexpr uint64_t kSlotTableOffset = 2048;   // the pack table; the unpack table follows it at capacity entries
static_assert(sizeof(SlotHeader) <= kSlotTableOffset, "the header must fit in front of the table");
enum { kSlotPlain = 0, kSlotXform = 1, kSlotStrided = 2, kSlotConvert = 3 };
// One launch over a slot's table by `wgs` persistent workgroups (a multiple of 8): the
// pipelined kernels of launch_copy_entries / launch_strided_entries / launch_xform_entries /
// launch_convert_entries with the entry count, blob positions and record shapes read from `hdr`.
// Same requirements: everything 16-byte aligned, entries of at most 4096 << sub_shift bytes
// (plain tables: sub_shift <= 3), less than 2 GiB per entry on the cache side.
hipError_t launch_slot(int kind, bool pack, const Chunk* chunks, const SlotHeader* hdr, uint32_t sub_shift,
                       uint8_t* const* layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
                       uint32_t n_layers, uint8_t* packed, uint64_t layer_stride, const XformDev& x,
                       uint32_t wgs, uint32_t* tickets, hipStream_t stream);

// Chunk launchers. max_wgs = 0: one workgroup per (4 KiB slice, layer), the fastest shape.
// max_wgs > 0: at most that many workgroups (a multiple of 8), striding over the same items,
// for a caller that wants the copy to leave part of the device to other kernels.
// policy: kPolicyTemporalLoads = plain instead of non-temporal loads, for a launch whose data may
// sit in the memory-side cache; kPolicyCachedStores = plain stores, for a launch whose output is
// read again while it still fits there (both ignored by a capped launch). tickets: a capped launch's block of counters
// (see launch_copy_entries), or nullptr; an uncapped launch ignores it and leaves it untouched. pipelined (launch_copy_chunks): a capped
// launch keeps the loads of its next trip in flight across the stores of the last one; for
// grids of at most 4 workgroups per CU (the kernel then needs more registers than 8 per CU fit).
hipError_t launch_strided_chunks(bool pack, const Chunk* chunks, uint32_t n_chunks,
                                 uint32_t sub_shift, uint8_t* const* layer_ptrs,
                                 uint32_t n_tensors, uint32_t first_layer, uint32_t n_layers,
                                 uint8_t* packed, uint64_t layer_stride, const BlobOffsets& blobs,
                                 const StrideTable& shapes, bool words, uint32_t max_wgs, uint32_t policy,
                                 uint32_t* tickets, hipStream_t stream);
// Converting gather (bf16 -> fp8 E4M3) of a chunk table, plain and strided chunks alike; lengths
// and packed positions count fp8 bytes, cache offsets and strides bytes of the bf16 cache.
hipError_t launch_convert_chunks(const Chunk* chunks, uint32_t n_chunks, uint32_t sub_shift,
                                 uint8_t* const* layer_ptrs, uint32_t n_tensors,
                                 uint32_t first_layer, uint32_t n_layers, uint8_t* packed,
                                 uint64_t layer_stride, const BlobOffsets& blobs,
                                 const StrideTable& shapes, uint32_t max_wgs, uint32_t* tickets,
                                 hipStream_t stream);
// A table of at most kSmallTable entries travels in the kernel arguments (2 KiB): a short
// request then needs no table upload, no upload event and no cross-stream wait before its
// first launch.
constexpr uint32_t kSmallTable = 64;
struct SmallTable {
  Chunk c[kSmallTable];
};
hipError_t launch_copy_chunks_small(bool pack, const SmallTable& table, uint32_t n_chunks,
                                    uint32_t sub_shift, uint8_t* const* layer_ptrs,
                                    uint32_t n_tensors, uint32_t first_layer, uint32_t n_layers,
                                    uint8_t* packed, uint64_t layer_stride,
                                    const BlobOffsets& blobs, uint32_t max_wgs, bool pipelined,
                                    uint32_t policy, uint32_t* tickets, hipStream_t stream);
hipError_t launch_copy_chunks(bool pack, const Chunk* chunks, uint32_t n_chunks,
                              uint32_t sub_shift, uint8_t* const* layer_ptrs, uint32_t n_tensors,
                              uint32_t first_layer, uint32_t n_layers, uint8_t* packed,
                              uint64_t layer_stride, const BlobOffsets& blobs, uint32_t max_wgs, bool pipelined,
                              uint32_t policy, uint32_t* tickets, hipStream_t stream);
// The capped launch of a plain table with 16-byte aligned entries (sub_shift 0 ... 3: at most
// 4 ... 32 KiB): `wgs` persistent workgroups (a multiple of 8), software-pipelined, one table
// entry per trip and workgroup (16 or 32 KiB) or per wavefront (4 or 8 KiB). Every address and
// length involved must be a multiple of 16.
hipError_t launch_copy_entries(bool pack, const Chunk* chunks, uint32_t n_chunks, uint32_t sub_shift,
                               uint8_t* const* layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
                               uint32_t n_layers, uint8_t* packed, uint64_t layer_stride,
                               const BlobOffsets& blobs, uint32_t wgs, uint32_t* tickets,
                               hipStream_t stream);
// ... of a table that travels in the kernel arguments (no tickets)
hipError_t launch_copy_entries_small(bool pack, const SmallTable& table, uint32_t n_chunks,
                                     uint32_t sub_shift, uint8_t* const* layer_ptrs, uint32_t n_tensors,
                                     uint32_t first_layer, uint32_t n_layers, uint8_t* packed,
                                     uint64_t layer_stride, const BlobOffsets& blobs, uint32_t wgs,
                                     hipStream_t stream);
// tickets (all the pipelined launchers): nine zeroed 32-bit counters 128 bytes apart that no other
// running launch uses, from which the workgroups take their work in order (they leave them
// zeroed again); nullptr: every workgroup strides through a fixed share of the work.
// The same pipeline for strided and for transposing tables (sub_shift 2 ... 7; larger entries
// are taken in parts of 16 or 32 KiB). Every entry must be 16-byte aligned on both sides, a multiple
// of 16 bytes long, and span less than 2 GiB on the cache side.
hipError_t launch_strided_entries(bool pack, const Chunk* chunks, uint32_t n_chunks, uint32_t sub_shift,
                                  uint8_t* const* layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
                                  uint32_t n_layers, uint8_t* packed, uint64_t layer_stride,
                                  const BlobOffsets& blobs, const StrideTable& shapes, uint32_t wgs,
                                  uint32_t* tickets, hipStream_t stream);
// ... strided tables with entries of 4 or 8 KiB (sub_shift 0 or 1): a wavefront per entry
hipError_t launch_strided_entries_by_wave(bool pack, const Chunk* chunks, uint32_t n_chunks, uint32_t sub_shift,
                                          uint8_t* const* layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
                                          uint32_t n_layers, uint8_t* packed, uint64_t layer_stride,
                                          const BlobOffsets& blobs, const StrideTable& shapes, uint32_t wgs,
                                          uint32_t* tickets, hipStream_t stream);
// ... and for the converting gather (entries a multiple of 16 elements long; sub_shift 0 ... 7,
// at sub_shift 0 a wavefront per entry).
hipError_t launch_convert_entries(const Chunk* chunks, uint32_t n_chunks, uint32_t sub_shift,
                                  uint8_t* const* layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
                                  uint32_t n_layers, uint8_t* packed, uint64_t layer_stride,
                                  const BlobOffsets& blobs, const StrideTable& shapes, uint32_t wgs,
                                  uint32_t* tickets, hipStream_t stream);
hipError_t launch_xform_entries(bool pack, const Chunk* chunks, uint32_t n_chunks, uint32_t sub_shift,
                                uint8_t* const* layer_ptrs, uint32_t n_tensors, uint32_t first_layer,
                                uint32_t n_layers, uint8_t* packed, uint64_t layer_stride,
                                const BlobOffsets& blobs, const XformDev& x, uint32_t wgs,
                                uint32_t* tickets, hipStream_t stream);
hipError_t launch_xform_chunks(bool pack, const Chunk* chunks, uint32_t n_chunks,
                               uint32_t sub_shift, uint8_t* const* layer_ptrs, uint32_t n_tensors,
                               uint32_t first_layer, uint32_t n_layers, uint8_t* packed,
                               uint64_t layer_stride, const BlobOffsets& blobs, const XformDev& x,
                               uint32_t max_wgs, uint32_t policy, uint32_t* tickets, hipStream_t stream);
// rows = workgroups striding over the 4 KiB slices of each range
hipError_t launch_copy_ranges(const void* src_base, void* dst_base, const int64_t* src_off,
                              const int64_t* dst_off, const int64_t* lens, int64_t n, int num_wg,
                              int rows, uint32_t max_wgs, hipStream_t stream);
// The same list through `wgs` persistent workgroups (a multiple of 8), a wavefront per range:
// the shape of a launch of many ranges, limited to a share of the device or not. walkers:
// ranges a wavefront moves side by side, 1, 2 or 4 (the copy; more for shorter ranges).
// share: a zeroed block of kShareBlockBytes that the launch may use until it has run (it leaves
// it zeroed), or nullptr. With it the ranges above kLongRange bytes (at most kShareMax of
// them, else none) are moved by all wavefronts together, in segments, instead of by the one
// wavefront each that meets them; not for the converting gather.
constexpr uint32_t kLongRange = 256u << 10, kShareMax = 500, kShareBlockBytes = 2048;
hipError_t launch_copy_ranges_persistent(bool convert, const void* src_base, void* dst_base,
                                         const int64_t* src_off, const int64_t* dst_off,
                                         const int64_t* lens, int64_t n, uint32_t wgs, int walkers,
                                         uint32_t* share, hipStream_t stream);
hipError_t launch_convert_ranges(const void* src_base, void* dst_base, const int64_t* src_off,
                                 const int64_t* dst_off, const int64_t* lens, int64_t n,
                                 int num_wg, int rows, uint32_t max_wgs, hipStream_t stream);
hipError_t launch_copy_linear(void* dst, const void* src, uint64_t bytes, hipStream_t stream);

}  // namespace kvt

#endif  // KVT_DEVICE_H_
