/*
 * kvt_hip.h -- C ABI of libkvt_hip.so: the MI355X (gfx950) implementation of
 * Blade-KVT's ParseBlock + block-copy (pack / unpack) path.
 *
 * Conventions
 *   - every function returns a KVT_* code (kvt_types.h); kvt_last_error() gives
 *     the message of the calling thread's most recent failure. No exception
 *     crosses this boundary.
 *   - hipStream_t / hipEvent_t travel as void* so that the header needs no HIP
 *     include; NULL stream = the device's default stream.
 *   - "cache offset" always means a byte offset relative to one layer tensor's
 *     base address, exactly like IpcBlock offsets in the reference.
 *   - every GPU entry point fails with KVT_ERR_NO_DEVICE when no gfx950 device
 *     is usable; there is no CPU fallback inside this library.
 *   - buffers handed to a launch whose extent the host knows (layer tensors at
 *     registration, the packed buffer of kvt_pack / kvt_unpack, both sides of
 *     the copy_handle_data calls, stager and object-ring transfers) are checked against what the
 *     runtime knows about the pointer: memory the device cannot address gives
 *     KVT_ERR_INVALID, an extent beyond the allocation holding the pointer
 *     KVT_ERR_OUT_OF_RANGE, instead of a GPU memory fault. Not checked inside a
 *     stream capture, nor where offsets live on the device (kvt_launch_copy_*).
 *   - threads: parsers, caches and plans are immutable once created and may be
 *     used from any number of threads at once (a plan may be launched on several
 *     streams); list containers (kvt_block_lists, kvt_run_lists), sessions and
 *     stagers belong to one thread at a time unless stated otherwise; an object
 *     ring locks itself.
 *
 * Each declaration cites the reference interface it replaces (paths relative
 * to the reference checkout).
 */
#ifndef KVT_HIP_H_
#define KVT_HIP_H_

#include "kvt_types.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------ misc */

const char* kvt_last_error(void);
/* sizeof() of the ABI structs as compiled, for binding self-checks:
 * which = 0 kvt_ipc_block, 1 kvt_worker_info, 2 kvt_task, 3 kvt_parse_opts,
 * 4 kvt_xform, 5 kvt_wire_layout, 6 kvt_run. */
uint64_t kvt_abi_sizeof(int which);
/* Number of usable gfx950 devices (0 when none / no driver). */
int kvt_device_count(void);

/* ---------------------------------------------------- ParseBlock (host) */

/* replaces compute_valid_ranks_pd()            kvtransfer/src/tx_stub.cpp:18-81 */
uint32_t kvt_compute_valid_ranks_pd(uint32_t p_tp, uint32_t d_tp, int32_t num_kv_heads);

/* replaces the per-destination dispatch of KvSendStub::TaskContext::
 * refresh_dst_info()                            kvtransfer/src/tx_stub.cpp:451-590
 * (valid ranks, effective kvt_tp_size / kvt_tp_rank, parser and TPKind).
 * KVT_ERR_UNSUPPORTED where the reference throws "unsupported cache_shape". */
int kvt_select_parser(int cache_shape, const kvt_worker_info* src, const kvt_worker_info* dst,
                      uint32_t* valid_mask, uint32_t* kvt_tp_size, uint32_t* kvt_tp_rank,
                      int* parser_id, int* tp_kind);

/* A compiled parser: the per-destination part of ParseBlock (all divisions,
 * strides and rank gating) resolved once, the way refresh_dst_info() picks a
 * ParseBlockFunc once per destination. */
/* Geometries the library declines: KVT_ERR_INVALID for more than 65536 tokens per block,
 * zero sizes and the like; KVT_ERR_OVERFLOW for a hybrid layout whose indexer block (tokens
 * per indexer block x indexer token size) reaches 4 GiB -- the reference forms that product in
 * 32 bits (kvtransfer/src/parse_block_qwen3_next.cpp:376-413) and emits wrapped ranges there. */
typedef struct kvt_parser kvt_parser;
int kvt_parser_create(int parser_id, const kvt_worker_info* src, const kvt_worker_info* dst,
                      uint32_t valid_mask, uint32_t kvt_tp_size, uint32_t kvt_tp_rank,
                      const kvt_parse_opts* opts, kvt_parser** out);
void kvt_parser_destroy(kvt_parser* p);

/* Growable per-tensor range lists: the C stand-in for the caller-owned
 * std::vector<std::vector<IpcBlock>>& send_blocks of ParseBlockFunc. */
typedef struct kvt_block_lists kvt_block_lists;
int kvt_block_lists_create(kvt_block_lists** out);
void kvt_block_lists_destroy(kvt_block_lists* l);
void kvt_block_lists_clear(kvt_block_lists* l);
uint32_t kvt_block_lists_num_tensors(const kvt_block_lists* l);
/* Borrowed view of tensor t's list; valid until the next mutation. */
int kvt_block_lists_view(const kvt_block_lists* l, uint32_t tensor, const kvt_ipc_block** data,
                         uint64_t* n);

/* Appends n caller-supplied ranges to tensor `tensor`'s list (growing the outer
 * size as needed). The receiving side uses it for the IpcBlock arrays that
 * arrive in a layer message                      kvtransfer/src/tcp_channel.cpp:190-221. */
int kvt_block_lists_append(kvt_block_lists* l, uint32_t tensor, const kvt_ipc_block* blocks,
                           uint64_t n);

/* replaces one ParseBlockFunc call              kvtransfer/include/parse_block_common.h:86-94
 * as issued per request by do_task()            kvtransfer/src/tx_stub.cpp:201-205.
 * APPENDS the task's ranges to `lists` (outer size grows to the parser's
 * tensor count). Errors: KVT_ERR_OUT_OF_RANGE where the reference throws
 * std::out_of_range (range validation of append_ipc_block_checked,
 * parse_block_common.h:31-68; bad block index), KVT_ERR_OVERFLOW for the
 * capacity overflow (parse_block_common.cpp:20-29). On error the lists keep
 * whatever was appended before the failing range, like the reference. */
int kvt_parse_block(const kvt_parser* p, const kvt_task* task, kvt_block_lists* lists);

/* ------------------------------------------- strided runs (device-side parse) */

/* Per-tensor lists of kvt_run. The TP-remapping parsers (P>D, P<D) produce one
 * range per token, per head, for K and V   kvtransfer/src/parse_block_common.cpp:81-129,
 *                                          kvtransfer/src/parse_block_flashinfer.cpp:82-235,
 *                                          kvtransfer/src/parse_block_qwen3_next.cpp:108-248
 * i.e. millions of 256-512 byte ranges for a large batch. kvt_parse_block_runs
 * emits the same sequence in closed form (one run per block segment), and a
 * plan built from runs evaluates the token -> offset arithmetic inside the
 * copy kernel instead of on the host. */
typedef struct kvt_run_lists kvt_run_lists;
int kvt_run_lists_create(kvt_run_lists** out);
void kvt_run_lists_destroy(kvt_run_lists* l);
void kvt_run_lists_clear(kvt_run_lists* l);
uint32_t kvt_run_lists_num_tensors(const kvt_run_lists* l);
int kvt_run_lists_view(const kvt_run_lists* l, uint32_t tensor, const kvt_run** data, uint64_t* n);
/* Appends runs that arrived from elsewhere (e.g. a peer that sends runs instead
 * of plain ranges). Runs with a zero count or length are refused. */
int kvt_run_lists_append(kvt_run_lists* l, uint32_t tensor, const kvt_run* runs, uint64_t n);
/* Number of ranges / bytes the runs of one tensor expand to. */
int kvt_run_lists_totals(const kvt_run_lists* l, uint32_t tensor, uint64_t* n_ranges,
                         uint64_t* n_bytes);
/* Same contract as kvt_parse_block (same ranges, same order, same errors), in
 * run form: expanding what this appends equals what kvt_parse_block appends. */
int kvt_parse_block_runs(const kvt_parser* p, const kvt_task* task, kvt_run_lists* lists);
/* Appends the expansion of every run to `out` (e.g. the range metadata of a
 * layer message for a peer that expects plain ranges). More than 2^31 ranges in
 * one tensor are refused (KVT_ERR_INVALID). */
int kvt_run_lists_expand(const kvt_run_lists* l, kvt_block_lists* out);
/* The inverse, for a receiver that got plain ranges: finds the arithmetic
 * progressions (innermost first, three levels) and appends runs whose expansion
 * is exactly the input list. */
int kvt_run_lists_compress(const kvt_block_lists* l, kvt_run_lists* out);

/* replaces merge_interval() + the erase of zero-length entries its callers do
 *                                               kvtransfer/src/channel.cpp:53-98,
 *                                               kvtransfer/src/tcp_channel.cpp:376-392
 * In place; returns the compacted count in *n_out and {min,max,total,count}
 * in stats (may be NULL). Sorting is stable on src_offset. */
int kvt_merge_interval(kvt_ipc_block* blocks, uint64_t n, uint64_t* n_out, uint64_t stats[4]);
/* Same, applied to every tensor of `lists` (what register_data does for PEQD). */
int kvt_block_lists_merge(kvt_block_lists* l);

/* replaces validate_ipc_block_bounds()          kvtransfer/src/channel.cpp:11-50
 * which: 0 = check src_offset, 1 = check dst_offset. *bad_idx (may be NULL)
 * receives the first offending index. */
int kvt_validate_ipc_block_bounds(const kvt_ipc_block* blocks, uint64_t n, uint64_t capacity,
                                  int which, uint64_t length_scale, uint64_t* bad_idx);

/* ------------------------------------------- registered cache (device) */

/* The `layers[layer][tensor]` base pointers Python hands to
 * init_kv_transfer_client                       kvtransfer/kvtransfer_pybind.cpp:131-199
 * (flattened by _flatten_cache,                 blade_kvt/hybrid_connector/kvtbackend.py:594-629).
 * ptrs is a host array of n_layers * n_tensors device pointers
 * (ptrs[layer * n_tensors + tensor]); capacity[t] is tensor t's size in bytes
 * (block_sizes[t] * layer_num_blocks). The table is copied to the device once.
 * Every pointer is checked against what the runtime knows about it: memory the
 * device cannot address is refused (KVT_ERR_INVALID), and so is a capacity that
 * reaches beyond the device allocation holding the pointer
 * (KVT_ERR_OUT_OF_RANGE) -- a kernel running off a tensor is a GPU memory
 * fault, not an error code. */
typedef struct kvt_cache kvt_cache;
int kvt_cache_register(int device, const void* const* ptrs, uint32_t n_layers, uint32_t n_tensors,
                       const uint64_t* capacity, kvt_cache** out);
void kvt_cache_destroy(kvt_cache* c);

/* --------------------------------------------------- copy plan (device) */

/* Optional intra-page layout transform applied while packing / unpacking.
 * KVT_XFORM_HND_NHD: the cache holds pages [2][heads][ntpb][row_bytes] (FlashInfer
 * HND) while the packed buffer holds them [2][ntpb][heads][row_bytes] (NHD).
 * Only valid for plans whose ranges are whole pages (page_bytes = 2 * heads *
 * ntpb * row_bytes, offsets and lengths multiples of it). The reference has no
 * layout-changing copy; this is an addition of this library. */
enum { KVT_XFORM_NONE = 0, KVT_XFORM_HND_NHD = 1 };
typedef struct kvt_xform {
  uint32_t kind;
  uint32_t heads;
  uint32_t ntpb;
  uint32_t row_bytes;
} kvt_xform;

/* A plan = the batch's merged range lists, split into bounded chunks and made
 * resident on the device once; every layer of the step replays it. Replaces
 * what IChannel::register_data() prepares      kvtransfer/src/tcp_channel.cpp:348-475
 * and the per-launch metadata upload of copy_handle_data_kernel_direct()
 *                                               kvtransfer/src/copy_kernels.cpp:363-439.
 *
 * `lists` is consumed as-is (call kvt_block_lists_merge first for PEQD).
 * src_capacity / dst_capacity: per-tensor byte sizes the ranges were validated
 * against; pack refuses a cache smaller than src_capacity, unpack one smaller
 * than dst_capacity. chunk_bytes bounds one table entry: a power of two in
 * [4096, 524288], or 0 for the largest size up to 32 KiB that leaves at most
 * 2 % of the launched workgroups without bytes to move. Every entry is served
 * by chunk_bytes / 4096 workgroups. The tables of a
 * plan of at most 64 entries (one short request) are passed to the kernel by
 * value: such a plan needs no upload and can be launched, or captured into a
 * graph, the moment it is created. */
typedef struct kvt_plan kvt_plan;
int kvt_plan_create(int device, const kvt_block_lists* lists, const uint64_t* src_capacity,
                    const uint64_t* dst_capacity, const kvt_xform* xform, uint32_t chunk_bytes,
                    kvt_plan** out);
/* May be called while launches of the plan are still queued: the table's storage
 * goes back into circulation only after the last of them has run, and the call
 * waits for nothing. A plan whose launches were recorded into a hipGraph must
 * outlive the last launch of that graph. */
void kvt_plan_destroy(kvt_plan* p);
/* A plan from runs: runs whose ranges are shorter than 4 KiB and 16-byte
 * aligned (offsets, strides, length) stay strided on the device (one table
 * entry per <= chunk_bytes of payload, the per-token arithmetic done by the
 * kernel); all others are expanded to plain chunks. Same pack / unpack entry
 * points and the same packed layout as a plan made from the expanded lists.
 * With 16-byte aligned layer base pointers, packed buffer, layer stride and blob
 * positions a strided entry moves one 16-byte vector per lane; 4-byte alignment
 * (a blob inside a layer message) is served by a slower word-wise path; anything
 * less is refused with KVT_ERR_INVALID. Every range of a run must fit the stated
 * capacities, and a run may not describe more bytes than the destination tensor
 * holds (its ranges are meant to be disjoint there): KVT_ERR_OUT_OF_RANGE. */
int kvt_plan_create_runs(int device, const kvt_run_lists* lists, const uint64_t* src_capacity,
                         const uint64_t* dst_capacity, uint32_t chunk_bytes, kvt_plan** out);
/* The same for a sender whose cache holds bf16 while the transfer buffer and the receiver
 * hold fp8 (BLLM_KVTRANS_BF162FP8_CONV: the P > D parsers then emit fp8 lengths, and
 * copy_d2h_bf16_to_fp8 converts while it gathers, kvtransfer/src/copy_kernels.cpp:733-959,
 * parse_block_common.cpp:81-129). The lists are what kvt_parse_block_runs produces with
 * kvt_parse_opts.bf16_to_fp8 set: every length counts fp8 bytes, i.e. elements; source offsets
 * and strides count bytes of the bf16 cache (they must be even), where 2 * length bytes are
 * read. kvt_pack converts (round to nearest even, saturating, like the launcher
 * kvt_launch_copy_d2h_bf16_to_fp8) with the per-token arithmetic still done by the kernel;
 * kvt_unpack scatters the fp8 bytes unchanged. A plain list goes through
 * kvt_run_lists_compress first. */
int kvt_plan_create_runs_bf16_to_fp8(int device, const kvt_run_lists* lists,
                                     const uint64_t* src_capacity, const uint64_t* dst_capacity,
                                     uint32_t chunk_bytes, kvt_plan** out);
/* Table entries that stayed strided (0 for a plan made from plain lists). */
uint64_t kvt_plan_num_strided_chunks(const kvt_plan* p);
/* Inspection without a GPU: a plan created with device = KVT_DEVICE_NONE keeps
 * its two tables on the host and cannot be launched. *chunks = 2 * n_chunks
 * entries of 32 bytes {u64 cache, u64 packed, u32 len, u16 tensor, u16 t0,
 * u32 shape, u32 0}: pack order first, then unpack order; *shapes = 16 record
 * shapes of 64 bytes {u32 vlen16, u32 inv, u32 n_inner, u32 inv_words, u64 outer[2],
 * u64 inner[2], u32 inv_inner, u32 0 x 3} ([0] source side, [1] destination side).
 * Entry semantics: see
 * csrc/kvt_device.h. Borrowed pointers, valid until the plan is destroyed. */
#define KVT_DEVICE_NONE (-1)
int kvt_plan_host_tables(const kvt_plan* p, const void** chunks, uint64_t* n_chunks,
                         uint32_t* chunk_bytes, const void** shapes);
/* The table upload is asynchronous; launches order themselves after it on
 * their stream. Host-blocking wait for it -- needed only before the plan is
 * used inside a stream capture (kvt_session_create does it itself). */
int kvt_plan_ready(const kvt_plan* p);
uint32_t kvt_plan_num_tensors(const kvt_plan* p);
uint64_t kvt_plan_num_chunks(const kvt_plan* p);
/* Packed bytes of tensor t in one layer (sum of its range lengths), and the
 * byte offset of its blob inside a layer's packed area (blobs are laid out
 * back to back, each start rounded up to 256 bytes). */
uint64_t kvt_plan_tensor_bytes(const kvt_plan* p, uint32_t tensor);
uint64_t kvt_plan_tensor_offset(const kvt_plan* p, uint32_t tensor);
/* Bytes one layer occupies in the packed buffer (incl. the rounding above). */
uint64_t kvt_plan_layer_bytes(const kvt_plan* p);

/* Pack = TCPChannel::send_data body             kvtransfer/src/tcp_channel.cpp:517-560
 * (+ RDMAStagedChannel::send_data               kvtransfer/src/rdma_staged_channel.cpp:246-265):
 * for layers [first_layer, first_layer + n_layers): tensor t's blob =
 * concatenation of cache[src_offset : +length] in list order, written to
 * packed + (layer - first_layer) * layer_stride + kvt_plan_tensor_offset(t).
 * One kernel launch for all requested layers; asynchronous on `stream`.
 * `packed` may be device memory or device-visible pinned host memory. */
int kvt_pack(const kvt_plan* p, const kvt_cache* cache, uint32_t first_layer, uint32_t n_layers,
             void* packed, uint64_t layer_stride, void* stream);

/* Unpack = TCPServer handle_kv_cache_data       kvtransfer/src/tcp_channel.cpp:190-261
 * (+ RDMAStagedServer                           kvtransfer/src/rdma_staged_server.cpp:441-463):
 * cache[dst_offset : +length] = next `length` bytes of the blob. */
int kvt_unpack(const kvt_plan* p, const kvt_cache* cache, uint32_t first_layer, uint32_t n_layers,
               const void* packed, uint64_t layer_stride, void* stream);

/* The same with caller-chosen blob positions: tensor t's blob of layer l lives at
 * base + (l - first_layer) * layer_stride + blob_offsets[t]. Used to pack
 * straight into a framed send buffer (blob_offsets from kvt_wire_layout) or to
 * unpack out of a received frame. 16-byte aligned positions take the vector
 * path; others fall back to 4-byte or byte copies. */
int kvt_pack_at(const kvt_plan* p, const kvt_cache* cache, uint32_t first_layer, uint32_t n_layers,
                void* base, uint64_t layer_stride, const uint64_t* blob_offsets, void* stream);
int kvt_unpack_at(const kvt_plan* p, const kvt_cache* cache, uint32_t first_layer,
                  uint32_t n_layers, const void* base, uint64_t layer_stride,
                  const uint64_t* blob_offsets, void* stream);

/* ------------------------------- plan slots: a new batch per replay of a graph */

/* A plan whose table lives at a FIXED device address and is refilled for every batch, so that
 * launches recorded once into a hipGraph (kvt_pack / kvt_unpack / kvt_session_save_layer inside
 * a stream capture) move a new batch on every replay. The reference builds a new range list for
 * every batch                                     kvtransfer/src/tx_stub.cpp:158-263 (do_task)
 * and sends it layer by layer                     kvtransfer/src/tx_stub.cpp:395-415,
 * with the per-layer event recorded every step    blade_kvt/kv_transfer_impl.py:319-327;
 * a plan made by kvt_plan_create names one batch for good, and a graph that holds its launches
 * can only ever replay that batch. A slot is the plan for an engine whose forward pass is a
 * replayed graph.
 *
 * What a recorded launch fixes: the slot (table address and capacity), the cache, the packed
 * buffer and its layer stride, the launch grid -- a slot is always served by persistent
 * workgroups, at most one or two per CU (fewer under kvt_set_copy_cu_usage as set when the
 * launch was recorded). What follows the batch: the number of table entries, where each
 * tensor's blob starts inside a packed layer and the blobs' sizes; the kernels read them from
 * a header in front of the table.
 *
 *   chunk_bytes      size of a table entry: a power of two, 4096 ... 32768 for plain slots
 *                    (0 = 32768), up to 524288 for transposing ones and for slots made for
 *                    runs (0 = 32768; a transposing slot holds at least one token row per entry)
 *   max_entries      table capacity per direction; a batch that needs more is refused
 *   max_layer_bytes  room of one layer in the packed buffer (what the launches check the
 *                    buffer against, and the smallest layer_stride accepted); a batch whose
 *                    packed layer is larger is refused. 0 = max_entries * chunk_bytes + 256 *
 *                    n_tensors, which no batch that fits the table exceeds
 * Everything a slot moves must be 16-byte aligned (range offsets and lengths, layer tensors,
 * packed buffer, layer stride): a batch that is not is refused by the fill, a cache or buffer
 * that is not by the launch. kvt_pack_at / kvt_unpack_at (caller-chosen blob positions) do
 * not take a slot. xform as for kvt_plan_create (may be NULL). */
typedef struct kvt_slot_layout {
  uint64_t n_entries;                       /* table entries the batch took                     */
  uint64_t layer_bytes;                     /* bytes of one packed layer of this batch          */
  uint32_t n_tensors, reserved0;
  uint64_t tensor_bytes[KVT_MAX_TENSORS];   /* what kvt_plan_tensor_bytes / _offset say of a    */
  uint64_t tensor_offset[KVT_MAX_TENSORS];  /* plan made from the same lists                    */
} kvt_slot_layout;
int kvt_plan_slot_create(int device, uint32_t n_tensors, const uint64_t* src_capacity,
                         const uint64_t* dst_capacity, const kvt_xform* xform, uint32_t chunk_bytes,
                         uint64_t max_entries, uint64_t max_layer_bytes, kvt_plan** out);
/* The same for batches in run form (kvt_parse_block_runs): strided table entries, the per-token
 * arithmetic done by the kernel; bf16_to_fp8 != 0 as kvt_plan_create_runs_bf16_to_fp8. A run
 * whose group of records (one token's K and V, or one record) is larger than chunk_bytes makes
 * the fill fail. */
int kvt_plan_slot_create_runs(int device, uint32_t n_tensors, const uint64_t* src_capacity,
                              const uint64_t* dst_capacity, uint32_t chunk_bytes, int bf16_to_fp8,
                              uint64_t max_entries, uint64_t max_layer_bytes, kvt_plan** out);
/* Puts a batch into the slot: `lists` as for kvt_plan_create (merged by the caller for PEQD; a
 * list container without tensors, or with empty lists, is an empty batch: launches then move
 * nothing and a session still signals every layer). The tables are built in pinned memory and
 * copied to the device asynchronously on `stream`: work queued on `stream` afterwards -- the
 * launch of the graph, normally -- sees the new batch, work queued before it the old one.
 * Launches on other streams: eager ones order themselves behind the fill (and the fill behind
 * them); a graph launched on another stream must be ordered by the caller. Never inside a
 * stream capture. Refused, with the slot's contents untouched: a batch that needs more than
 * max_entries entries or max_layer_bytes per layer (KVT_ERR_OUT_OF_RANGE), ranges outside the
 * capacities given at creation (KVT_ERR_OUT_OF_RANGE), ranges that are not 16-byte aligned
 * (KVT_ERR_INVALID). The host may run ahead of the device by one fill without blocking; a third
 * fill waits until the first one's copy has run. *layout (may be NULL) receives where the
 * blobs of this batch lie; kvt_plan_tensor_bytes / _offset / _layer_bytes / _num_chunks of the
 * slot answer for the newest fill. One thread at a time fills a slot. */
int kvt_plan_slot_fill(kvt_plan* slot, const kvt_block_lists* lists, void* stream,
                       kvt_slot_layout* layout);
int kvt_plan_slot_fill_runs(kvt_plan* slot, const kvt_run_lists* lists, void* stream,
                            kvt_slot_layout* layout);

/* ------------------------------------------ layer-message framing (host) */

/* The per-layer messages of the staged transports:
 *   KVT_WIRE_TCP          TCPChannel::send_data / TCPServer::handle_kv_cache_data
 *                                               kvtransfer/src/tcp_channel.cpp:477-560, 141-261
 *   KVT_WIRE_RDMA_STAGED  RDMAStagedChannel::send_data / RDMAStagedServer
 *                                               kvtransfer/src/rdma_staged_channel.cpp:246-300,
 *                                               kvtransfer/src/rdma_staged_server.cpp:379-420
 * Byte layout: see csrc/kvt_wire.cpp. Integers are host-endian 64-bit like the
 * reference's size_t memcpy's. */
enum { KVT_WIRE_TCP = 0, KVT_WIRE_RDMA_STAGED = 1 };
#define KVT_WIRE_MAGIC 0x4B564361u /* KV_CACHE_DATA_MAGIC, kvtransfer/include/copy_utils.h:32 */
typedef struct kvt_wire_layout {
  uint64_t total_bytes;
  uint32_t n_tensors;
  uint32_t reserved0;
  uint64_t meta_offset[KVT_MAX_TENSORS]; /* where tensor t's [n][ranges] starts */
  uint64_t blob_offset[KVT_MAX_TENSORS];
  uint64_t blob_bytes[KVT_MAX_TENSORS];
} kvt_wire_layout;
/* Sizes and positions of a frame for these range lists (the total_bytes sum of
 * register_data,                                kvtransfer/src/tcp_channel.cpp:431-446). */
int kvt_wire_layout_of(int format, const kvt_block_lists* lists, kvt_wire_layout* out);
/* Writes header and range metadata; the blob areas are left for the pack. */
int kvt_wire_write_frame(int format, void* buf, uint64_t capacity, uint64_t reqid,
                         uint64_t layer_idx, const kvt_block_lists* lists, kvt_wire_layout* out);
/* Receiver side: checks magic, truncation and sizes the way the reference's
 * handlers do, fills `lists` with the ranges and `out` with the blob positions.
 * expect_tensors = 0 accepts any count. Errors: KVT_ERR_INVALID. */
int kvt_wire_parse_frame(int format, const void* buf, uint64_t len, uint32_t expect_tensors,
                         uint64_t* reqid, uint64_t* layer_idx, kvt_block_lists* lists,
                         kvt_wire_layout* out);

/* ------------------------------------------------- KVStore block objects */

/* Range lists whose packed blob is a sequence of per-block store objects, in
 * the order of the given block ids: the object of block b is what
 * FileBackend saves / loads per (block hash, rank, layer),
 * `kvcache[:, b]` for the [2, nblk, bs, h, d] layout
 *                                               blade_kvt/hybrid_connector/file_backend.py:222-232, 269-283
 * (K block then V block), and the contiguous block for block-major layouts.
 * Object i of tensor t starts at i * block_sizes[t] inside that tensor's blob.
 * Do not merge these lists. *object_bytes = sum over tensors of the block size. */
int kvt_block_object_lists(int cache_shape, const kvt_worker_info* src, const kvt_worker_info* dst,
                           const uint32_t* src_blocks, const uint32_t* dst_blocks, uint64_t n,
                           kvt_block_lists* lists, uint64_t* object_bytes);

/* A plan whose packed side holds one object per block SPANNING ALL LAYERS, for a
 * store that keeps a block under one key (MooncakeKVSBackend saves whole blocks,
 * all layers at once, when the last layer is done,
 *                                               blade_kvt/hybrid_connector/mooncake_kvsbackend.py:382-437).
 * `lists` = kvt_block_object_lists output (one cache tensor per layer), object_bytes
 * = its *object_bytes, object_stride >= n_layers * object_bytes. Packed with
 * layer_stride = object_bytes, block i's object is
 *   [layer 0 part][layer 1 part]... at base + i * object_stride,
 * each part being the per-layer object described above. (The store library is
 * third-party and not part of the reference checkout; the order of the parts
 * inside an object is this library's choice.) kvt_plan_layer_bytes() = the span
 * of one layer's parts: (n_objects - 1) * object_stride + object_bytes. */
int kvt_plan_create_objects(int device, const kvt_block_lists* lists, const uint64_t* src_capacity,
                            const uint64_t* dst_capacity, uint64_t object_bytes,
                            uint64_t object_stride, uint32_t chunk_bytes, kvt_plan** out);

/* The store's block ids -> the engine's kernel-block ids when one store block
 * spans `factor` kernel blocks: out[i] = ids[i / factor] * factor + i % factor
 * for i < n * factor (VineyardKVSBackend._enlarge_list,
 *                                               blade_kvt/hybrid_connector/kvsbackend.py:207-214). */
int kvt_enlarge_block_ids(const uint32_t* ids, uint64_t n, uint32_t factor, uint32_t* out);

/* --------------------------- drop-ins for the reference copy entry points */

/* replaces launch_copy_d2h_direct_kernel()      kvtransfer/src/copy_kernels.cu:268-281
 * gather: dst[dst_offsets[i] : +lengths[i]] = gpu_src_base[src_offsets[i] : ...].
 * The three arrays live in device memory. num_wg / threads_per_wg <= 0 pick
 * this library's launch shape. A long list is moved by persistent workgroups, a wavefront per
 * range; ranges above 256 KiB (up to 500 of them per launch) are listed by a small kernel in
 * front and moved by all wavefronts together at the end, so that a list which mixes many short
 * ranges with a few very long ones (merged runs of hundreds of MiB) does not wait for single
 * wavefronts. */
int kvt_launch_copy_d2h_direct(const void* gpu_src_base, void* dst, const int64_t* src_offsets,
                               const int64_t* dst_offsets, const int64_t* lengths, int64_t n,
                               int num_wg, int threads_per_wg, void* stream);
/* replaces launch_copy_h2d_direct_kernel()      kvtransfer/src/copy_kernels.cu:179-192 */
int kvt_launch_copy_h2d_direct(const void* src, void* gpu_dst_base, const int64_t* src_offsets,
                               const int64_t* dst_offsets, const int64_t* lengths, int64_t n,
                               int num_wg, int threads_per_wg, void* stream);
/* replaces launch_copy_d2h_bf16_to_fp8_kernel() kvtransfer/src/copy_kernels.cu:467-481
 * lengths are ELEMENT counts, src offsets in bf16 bytes, dst offsets in fp8 bytes. */
int kvt_launch_copy_d2h_bf16_to_fp8(const void* gpu_src_base, void* dst,
                                    const int64_t* src_offsets, const int64_t* dst_offsets,
                                    const int64_t* lengths, int64_t n, int num_wg,
                                    int threads_per_wg, void* stream);

/* replaces env_kernel_copy_sm_usage(), BLLM_KVTRANS_KERNEL_COPY_SM_USAGE
 *                                               kvtransfer/src/envcfg.cpp:311-326,
 * as CopyKernelConfig::initialize applies it    kvtransfer/src/copy_kernels.cpp:327-335
 * (blocks of a copy launch = resident blocks per SM x SMs x usage): the share of the
 * device's CUs a copy launch may occupy, for an engine that overlaps transfers with its
 * forward pass. usage in (0, 1]; 1 (the default) keeps one workgroup per 4 KiB slice, the
 * fastest shape. Below 1 every copy launch of this library on `device` (plans, sessions,
 * stagers, the launchers below) runs as at most usage x CUs x 8 persistent 256-lane
 * workgroups, rounded down to a multiple of 8 and at least 8, that stride over the same
 * work; results are identical. Takes effect for launches issued after the call (a launch
 * captured into a graph keeps the shape it was captured with). Passing num_wg > 0 to a
 * launcher still bounds that launch further.
 * The first call with usage < 1 for a device allocates 2 MiB of device memory there (blocks
 * of counters from which the persistent workgroups of a launch take their work in order; a
 * launch borrows one until it has run; the launches of a plan that are recorded into one
 * stream capture on one stream share one, which stays with the plan until it is destroyed;
 * 256 of the device's 1024 blocks are kept for captures): call it at start-up, not inside a
 * stream capture. A graph that holds limited launches must not run at the same time as a
 * second instantiation of itself. */
int kvt_set_copy_cu_usage(int device, double usage);
/* The current setting and the workgroup limit it stands for (0 = none); either may be NULL. */
int kvt_get_copy_cu_usage(int device, double* usage, uint32_t* max_workgroups);
/* Counters of the launches limited to a CU share that wanted a block of work counters, since
 * the first kvt_set_copy_cu_usage(device, < 1): out[0] eager launches that got one, out[1] eager
 * launches that found none free (they ran with a fixed stride per workgroup instead: slower,
 * same result), out[2] blocks handed to stream captures (one per plan, capture and stream), out[3]
 * launches recorded into a capture that found none. */
int kvt_get_copy_ticket_stats(int device, uint64_t out[4]);

/* No counterpart in the reference (its copy kernel uses one load flavour). A pack / unpack
 * launch whose payload (bytes moved one way, all layers of the launch) is at most
 * payload_bytes reads with plain loads, a larger one with non-temporal loads. Default: 0,
 * non-temporal loads always -- they are the faster ones whenever a launch's data is read
 * once, whether it comes from HBM or was left in the 256 MiB memory-side cache by the kernel
 * that produced it (MI355X, one request per launch, 32 to 256 MiB: 1 to 6 % faster on
 * uncached data, 2 to 22 % faster right behind a producer). Plain loads pay when the SAME data
 * is read again while it is still cached (one layer gathered for several destinations, blocks
 * stored and sent): the second reader then hits, 64 / 128 / 256 MiB of payload back to back:
 * +12 / +7 / +8 % (pack), +18 / +26 / +22 % (unpack); beyond 256 MiB they lose again. A caller
 * with such a pattern sets the limit to the largest launch it repeats. Process-wide; takes
 * effect for launches issued after the call (a launch captured into a graph keeps what it was
 * captured with). Results are identical either way. */
int kvt_set_copy_cached_load_max(uint64_t payload_bytes);
uint64_t kvt_get_copy_cached_load_max(void);
/* The same for the stores (no counterpart in the reference either): a pack / unpack launch
 * between device buffers whose payload is at most payload_bytes writes with plain stores, which
 * leave their lines in the memory-side cache, instead of non-temporal write-through ones. For a
 * caller whose next launch reads what this one wrote while it still fits there (a request packed
 * and unpacked on the same GPU, a blob packed and at once stored and sent). Default: 0, never.
 * Process-wide, for launches issued after the call; launches limited to a CU share and launches
 * whose packed side is pinned host memory keep the streaming stores. Results are identical. */
int kvt_set_copy_cached_store_max(uint64_t payload_bytes);
uint64_t kvt_get_copy_cached_store_max(void);

/* replaces launch_copy_int64_array_h2d_kernel()  kvtransfer/src/copy_kernels.cu:93-103
 * (declared for the channels, kvtransfer/src/copy_kernels.cpp:101-108): a kernel reads
 * num_elements int64 from pinned (device-visible) host memory and writes them to device_dst,
 * the metadata upload without a DMA copy. num_wg / threads_per_wg are accepted and ignored. */
int kvt_launch_copy_int64_array_h2d(const int64_t* host_src, int64_t* device_dst,
                                    int64_t num_elements, int num_wg, int threads_per_wg,
                                    void* stream);

/* replaces BLLM_KVTRANS_COPY_MEMCPY_BLOCK_THRESHOLD_BYTES / BLLM_KVTRANS_COPY_MEMCPY_MAX_BLOCKS
 *                                               kvtransfer/src/copy_kernels.cpp:157-158, 496-499,
 * the static part of select_copy_method()       kvtransfer/src/copy_kernels.cpp:610-617:
 * kvt_copy_handle_data_with_kernel hands a list to the DMA engines (one copy per range) when it
 * has at most max_ranges ranges and every range is at least min_range_bytes long; in a longer or
 * mixed list whose lengths differ, the ranges of at least min_range_bytes still go there one by
 * one and the kernel moves the rest (enqueue_hybrid_copy, copy_kernels.cpp:675-722). Defaults:
 * 8 MiB and 16, measured on one MI355X box against pinned host memory (the reference's
 * defaults, 256 KiB and 16, suit a part whose copy kernel is slower across PCIe than this
 * one's). They are the rule until kvt_initialize_copy_method_profile has measured the box at
 * hand, and for good once they have been set through this call (both directions at once).
 * max_ranges = 0 switches the DMA route off. Process-wide. */
int kvt_set_copy_memcpy_thresholds(uint64_t min_range_bytes, uint64_t max_ranges);
int kvt_get_copy_memcpy_thresholds(uint64_t* min_range_bytes, uint64_t* max_ranges);
/* Undoes kvt_set_copy_memcpy_thresholds: the defaults again, and the start-up measurement in
 * charge again where it has run. */
int kvt_reset_copy_memcpy_thresholds(void);

enum { KVT_COPY_H2D = 0, KVT_COPY_D2H = 1 };
/* replaces initialize_copy_method_profile()     kvtransfer/include/copy_kernels.h:15-22,
 *                                               kvtransfer/src/copy_kernels.cpp:495-591, 724-728
 * (called once per copy thread, kvtransfer/src/copy_utils.cpp:52). Checks that `device` is a
 * usable gfx950 part, looks up the address of that device's static metadata array (see
 * kvt_copy_handle_data_kernel_direct_static) and, on the first call of the process, times
 * loops of DMA copies against the copy kernel on pinned host memory in both directions (8
 * ranges of 256 KiB and 2 of 16 MiB by either route). From then on, unless the thresholds
 * above have been set by the caller, kvt_copy_handle_data_with_kernel routes a list of n
 * ranges and `total` bytes by comparing n * dma_fixed + total * dma_per_byte with kernel_fixed
 * + total * kernel_per_byte (select_copy_method, copy_kernels.cpp:593-619, which looks the
 * list up in a table of measured buckets), and in a list of mixed lengths gives a range a DMA
 * copy of its own when that beats the kernel's cost per byte for it (select_single_block_method,
 * :621-631). Allocates and frees 32 MiB of pinned and of device memory and blocks for a few
 * tens of milliseconds: call it at start-up, not in a serving loop. */
int kvt_initialize_copy_method_profile(int device);
/* What the start-up measurement found for `direction` (*measured = 0 and zeros before it has
 * run): microseconds per DMA copy and per MiB moved by it, per kernel launch (metadata upload
 * included) and per MiB moved by it; the shortest range that gets a DMA copy of its own in a
 * mixed list under the rule in force (~0: none); the time the measurement took. Any pointer
 * may be NULL. */
int kvt_get_copy_method_profile(int direction, double* dma_fixed_us, double* dma_us_per_mib,
                                double* kernel_fixed_us, double* kernel_us_per_mib,
                                uint64_t* single_range_min_bytes, int* measured, double* elapsed_ms);
/* replaces get_kernel_copy_buffer()             kvtransfer/include/copy_utils.h:127,
 *                                               kvtransfer/src/copy_utils.cpp:9-57,137-146
 * The calling THREAD's metadata buffers for kvt_copy_handle_data_with_kernel: device and
 * pinned host memory of 3 * 8 * max_block_num bytes each (max_block_num <= 0: 8192), one pair
 * per (thread, device), created on first use and released when the thread ends. Asking for
 * MORE ranges on the same device replaces the pair, after the thread's two streams have
 * drained: the pointers handed out before are invalid from then on (the reference sizes its
 * buffers once from the environment and never regrows). A request for another device, or for
 * a stream, leaves them alone. */
int kvt_get_kernel_copy_buffer(int device, int64_t max_block_num, int64_t** dev_meta,
                               int64_t** host_meta);
/* replaces get_thread_local_h2d_stream() / get_thread_local_d2h_stream()
 *                                               kvtransfer/src/copy_utils.cpp:59-95,148-154
 * direction = KVT_COPY_H2D / KVT_COPY_D2H: the calling thread's non-blocking stream for that
 * direction on `device` (the reference's live on the device of the thread's buffers). The
 * handle stays valid until the thread ends, whatever buffers or devices the thread asks for
 * in between. */
int kvt_get_thread_local_stream(int device, int direction, void** stream);
/* replaces copy_handle_data_with_kernel()       kvtransfer/include/copy_kernels.h:87-97,
 *                                               kvtransfer/src/copy_kernels.cpp:733-827
 * Same calling convention: blocks[i].dst_offset is the GPU-side offset for BOTH
 * directions, the contiguous side advances by blocks[i].length (running sum),
 * tensor_data_size must equal the sum of lengths. dev_meta / host_meta are the
 * caller's metadata buffers (>= 3 * 8 * max_block_num bytes each, host_meta
 * pinned); more than max_block_num ranges are processed in batches with a
 * stream synchronisation after each, like the reference. max_block_num <= 0
 * means 8192 (BLLM_KVTRANS_KERNEL_COPY_MAX_BLOCK_NUM's default).
 * A single batch is only enqueued, like the reference's: host_meta (and dev_meta)
 * must stay untouched until `stream` has run the copy, so a thread that reuses its
 * buffers for the next call waits for the stream first.
 * Like the reference's, this entry point may decide against its kernel and hand
 * the list, or the longest ranges of a mixed list, to the DMA engines, one
 * hipMemcpyAsync per range on `stream` (select_copy_method / enqueue_hybrid_copy,
 * copy_kernels.cpp:621-722): by the cost model of kvt_initialize_copy_method_profile
 * once that has run, before that (or when the caller has set them) by the
 * thresholds of kvt_set_copy_memcpy_thresholds: at most 16 ranges of at least
 * 8 MiB each. */
int kvt_copy_handle_data_with_kernel(void* tensor_buf, void* layer_gpu_ptr,
                                     const kvt_ipc_block* blocks, uint64_t n,
                                     uint64_t tensor_data_size, int direction, int device,
                                     void* stream, int64_t* dev_meta, int64_t* host_meta,
                                     int64_t max_block_num);
/* replaces copy_handle_data_kernel_direct()     kvtransfer/include/copy_kernels.h:24-57,
 *                                               kvtransfer/src/copy_kernels.cpp:363-439
 * One batch, no internal synchronisation: the three device arrays (n int64 each)
 * and host_meta (3 n int64, pinned) belong to the caller and must stay untouched
 * until the stream has run the copy. With use_explicit_host_offsets the
 * contiguous-side offset of range i is blocks[i].src_offset instead of the
 * running sum. Unlike the reference (which only asserts), ranges that leave
 * the contiguous buffer are refused with KVT_ERR_OUT_OF_RANGE. */
int kvt_copy_handle_data_kernel_direct(void* tensor_buf, void* layer_gpu_ptr,
                                       const kvt_ipc_block* blocks, uint64_t n,
                                       uint64_t tensor_data_size, int direction, int device,
                                       void* stream, int64_t* src_offsets_dev,
                                       int64_t* dst_offsets_dev, int64_t* lengths_dev,
                                       int64_t* host_meta, int use_explicit_host_offsets);
/* No counterpart in the reference. kvt_copy_handle_data_kernel_direct for callers that cannot
 * allocate device memory or hand over a device workspace (code under hipGraph capture, tight
 * serving loops, harnesses that forbid hipMalloc): the three device-side metadata arrays live
 * in a 192 KiB array that is part of the library's code object (one copy per GPU, held until
 * the process ends), so the caller passes inputs, outputs and the pinned host_meta staging
 * area (3 n int64) only. The call allocates and frees nothing, on the host side of the
 * runtime or the device: the metadata is brought over by a copy kernel reading host_meta.
 * At most 8192 ranges per call: more are refused with KVT_ERR_INVALID. All calls on one GPU
 * share that GPU's array, which keeps the last call's metadata until the next one overwrites
 * it. Eager calls are kept apart by the library: each makes its stream wait for the previous
 * call on that GPU (whatever stream that was on, through one event per GPU created at
 * kvt_initialize_copy_method_profile or the first call), so copy threads with a stream each
 * (kvtransfer/src/copy_utils.cpp:59-95) may call it at will and their copies run one after the
 * other. Calls recorded into a stream capture are ordered by their graph alone: two graphs
 * that hold such calls, or one graph launched twice at once, must not run at the same time,
 * nor beside an eager call. host_meta must stay untouched until the stream has run the copy.
 * Errors as kvt_copy_handle_data_kernel_direct. */
int kvt_copy_handle_data_kernel_direct_static(void* tensor_buf, void* layer_gpu_ptr,
                                              const kvt_ipc_block* blocks, uint64_t n,
                                              uint64_t tensor_data_size, int direction, int device,
                                              void* stream, int64_t* host_meta,
                                              int use_explicit_host_offsets);
/* replaces copy_d2h_bf16_to_fp8()               kvtransfer/include/copy_kernels.h:112-121,
 *                                               kvtransfer/src/copy_kernels.cpp:833-959
 * blocks[i].length = bf16 bytes at the source; the contiguous side receives
 * length / 2 fp8 (E4M3, round-to-nearest-even, saturating) bytes per range. */
int kvt_copy_d2h_bf16_to_fp8(void* tensor_buf, const void* layer_gpu_ptr,
                             const kvt_ipc_block* blocks, uint64_t n, uint64_t tensor_data_size,
                             int device, void* stream, int64_t* dev_meta, int64_t* host_meta,
                             int64_t max_block_num);

/* ------------------------------------- per-layer gating on a side stream */

/* Replaces Step / StepGuard / CudaEventBarrier  kvtransfer/include/step.h, src/step.cpp:49-69,
 *                                               kvtransfer/src/context.cpp:18-20
 * and the host-side wait in do_send()           kvtransfer/src/tx_stub.cpp:395-415:
 * the reference parks a host thread in cudaEventSynchronize per layer; here the
 * dependency stays on the device (event record on the compute stream, stream
 * wait on a side stream, pack launch), so the sequence can be captured into a
 * hipGraph together with the forward pass. Completion of a layer's pack is published by the
 * device itself (a one-lane kernel behind the pack bumps a per-layer counter mirrored in
 * pinned host memory); the transport thread's wait polls that word. The signal is therefore
 * the same for eagerly issued and for replayed (graph) sequences, and a wait touches neither
 * an event nor a stream.
 *
 * Steps. A session serves any number of forward passes ("steps", Step objects in the
 * reference). kvt_session_begin_step starts one; a session that only ever serves one step
 * needs no call (the first save_layer begins step 1). The last 8 steps are tracked, i.e. the
 * transport may lag up to 7 steps behind the forward pass. */
typedef struct kvt_session kvt_session;
int kvt_session_create(const kvt_plan* plan, const kvt_cache* cache, void* packed,
                       uint64_t layer_stride, kvt_session** out);
/* Wakes threads parked in a wait (they return KVT_ERR_INVALID), waits for them to leave and
 * for the side stream to drain. */
void kvt_session_destroy(kvt_session* s);
/* The next batch on the same session: packs issued from here on use `plan` and write to
 * `packed` (stream, events and counters of a session are not cheap to create; a sender keeps
 * one session per destination and gives it each batch's plan). Layers already issued keep
 * what they were issued with. Refused once save_layer calls of this session have been captured
 * into a graph (the graph would go on launching the old plan) -- unless the session was made
 * with a plan slot and is given the same slot, buffer and stride again: such a session takes
 * its next batch through kvt_plan_slot_fill, captured or not, and needs no call here. Call it
 * from the thread that drives the forward pass, between steps. */
int kvt_session_set_plan(kvt_session* s, const kvt_plan* plan, void* packed, uint64_t layer_stride);
/* Host only, never captured: starts step *step (1, 2, ...). Eager use: call before the step's
 * first save_layer. Graph use: call before EACH launch of a graph that holds captured
 * save_layer calls -- the layers recorded in it count as submitted from here on, so launch
 * the graph next. `step` may be NULL. */
int kvt_session_begin_step(kvt_session* s, uint64_t* step);
/* save_kv_layer hook: layer `layer` of the cache is complete once the work
 * already queued on compute_stream has run. Never blocks the host. Capturable: inside a
 * stream capture nothing runs, the layer's pack and its completion signal become part of
 * the graph. A failure (refused launch, HIP error) is latched in the current step: threads
 * waiting for that step return it instead of waiting on. */
int kvt_session_save_layer(kvt_session* s, uint32_t layer, void* compute_stream);
/* The same for layers [first_layer, first_layer + n_layers) at once (no counterpart in the
 * reference, which signals every layer by itself): they are complete once the work already
 * queued on compute_stream has run, and are packed by ONE launch behind one event. A caller
 * whose step is bound by the host (an eagerly issued event hop between two streams costs
 * 16-19 us of host time on MI355X, whatever the launch moves) calls this once per group of
 * layers instead of kvt_session_save_layer per layer; the transport still waits per layer, and
 * the layers of a group become ready together. */
int kvt_session_save_layers(kvt_session* s, uint32_t first_layer, uint32_t n_layers,
                            void* compute_stream);
/* The same without the hop (no counterpart in the reference): the layers are packed on
 * compute_stream itself, behind whatever is queued there, and whatever the caller queues next
 * on that stream runs after the pack. For the last layer(s) of a step, when no further compute
 * is left for the pack to overlap with: what the transport waits for after the forward pass
 * then ends one launch behind the last layer's compute instead of one cross-stream hop
 * (18-27 us on MI355X) behind it. Signals, steps and errors as kvt_session_save_layers;
 * kvt_session_join does not wait for these launches (they are on the caller's stream
 * already). Capturable. */
int kvt_session_save_layers_inline(kvt_session* s, uint32_t first_layer, uint32_t n_layers,
                                   void* compute_stream);
/* The same for a caller that owns the per-layer events, as the reference's Python side does:
 * it creates one event per layer, hands their handles to the library at init and records
 * event[layer] itself after the layer's KV is written (blade_kvt/kv_transfer_impl.py:287-291,
 * 320-327; consumed by CudaEventBarrier::wait, kvtransfer/src/context.cpp:18-20).
 * `ready_event` is that hipEvent_t (torch.cuda.Event.cuda_event), already recorded on the
 * compute stream; the side stream waits for it, the host never does. */
int kvt_session_save_layer_event(kvt_session* s, uint32_t layer, void* ready_event);
/* Host-blocking wait until the packed bytes of `layer` in step `step` are complete (what the
 * transport thread calls before send_data(layer), Step::wait_layer_ready in the
 * reference, kvtransfer/src/step.cpp:49-69). May be called from any thread and before the
 * step has begun or the layer has been submitted: it then waits for that first. Issues no
 * HIP call and synchronises nothing but the calling thread. step = 0: the newest step.
 * Errors: the latched failure of the step; KVT_ERR_INVALID when the step is no longer tracked
 * or the session is being destroyed. A layer that the step never submits is waited for
 * until the session is destroyed, like the reference's. */
int kvt_session_wait_layer_step(kvt_session* s, uint64_t step, uint32_t layer);
/* The same with a limit (no counterpart in the reference, whose wait has none): returns
 * KVT_ERR_TIMEOUT when the layer is not complete within timeout_us microseconds -- the step
 * has not begun, the layer has not been submitted, or the GPU has not got to it. Nothing
 * about the step changes; the wait can simply be repeated. For transport threads that must
 * notice a shutdown or a stalled device between waits. */
int kvt_session_wait_layer_for(kvt_session* s, uint64_t step, uint32_t layer, uint64_t timeout_us);
/* kvt_session_wait_layer_step(s, 0, layer). */
int kvt_session_wait_layer(kvt_session* s, uint32_t layer);
/* Makes `stream` wait for every pack issued so far (joins the side stream
 * back; required before ending a capture that included save_layer calls). */
int kvt_session_join(kvt_session* s, void* stream);
/* hipStream_t of the side stream (for tests / profiling). Threads: begin_step / save_layer /
 * join from the thread that drives the forward pass, the waits from any thread. */
void* kvt_session_side_stream(kvt_session* s);

/* ------------------------------------ pinned-host staging (KVStore path) */

/* A ring of pinned host slots fed by hipMemcpyAsync on a copy stream of the library's, so
 * that D2H of layer L overlaps the pack of layer L+1 (and H2D of L+1 overlaps
 * the unpack of L). The copy streams are four per device, made together with the first
 * stager, kept until the process ends and handed to the stagers in turn: stagers made one
 * after the other (a saving and a loading one) then copy through different hardware queues,
 * which is what lets the two directions overlap; from the fifth on stagers share streams.
 * Stands where the reference's KVStore backends hand packed
 * layers to a host-side store                   blade_kvt/hybrid_connector/kvsbackend.py:268-357,
 *                                               blade_kvt/hybrid_connector/file_backend.py:222-283.
 * slot_bytes bounds one transfer; n_slots >= 2. One stager serves one caller
 * thread at a time (save / load calls of different threads must not overlap);
 * a saving and a loading side each take their own stager. */
typedef struct kvt_stager kvt_stager;
int kvt_stager_create(int device, uint64_t slot_bytes, uint32_t n_slots, kvt_stager** out);
void kvt_stager_destroy(kvt_stager* s);
void* kvt_stager_slot(kvt_stager* s, uint32_t slot);
void* kvt_stager_copy_stream(kvt_stager* s);
/* Device -> slot: waits (on the copy stream) for everything queued on
 * `producer_stream`, then copies `bytes` from dev into the slot. */
int kvt_stager_save(kvt_stager* s, uint32_t slot, const void* dev, uint64_t bytes,
                    void* producer_stream);
/* Same, to byte `slot_offset` of the slot (e.g. the blob area of a frame). */
int kvt_stager_save_at(kvt_stager* s, uint32_t slot, uint64_t slot_offset, const void* dev,
                       uint64_t bytes, void* producer_stream);
/* Slot -> device on the copy stream, then makes consumer_stream wait for it. The copy
 * itself first waits for everything queued on consumer_stream so far (the device buffer may
 * still be read there). A caller that alternates between two device buffers therefore gives
 * each its own consumer stream: on a shared one the copy for one buffer would also wait for
 * the kernels reading the other, and transfer and kernels would take turns (about 2 % of the
 * PCIe rate for 1 GiB transfers). */
int kvt_stager_load(kvt_stager* s, uint32_t slot, void* dev, uint64_t bytes,
                    void* consumer_stream);
int kvt_stager_load_at(kvt_stager* s, uint32_t slot, uint64_t slot_offset, void* dev,
                       uint64_t bytes, void* consumer_stream);
/* Host-blocking: the slot's last save/load has completed. */
int kvt_stager_wait(kvt_stager* s, uint32_t slot);
/* Measured plain pinned<->device copy rate in bytes/s (direction: KVT_COPY_*),
 * the ceiling the staging path is reported against. */
int kvt_measure_pcie(int device, int direction, uint64_t bytes, uint32_t repeats,
                     double* bytes_per_s);

/* The same with both directions running at the same time on two streams (a saving and a
 * loading stager side by side): the rate each direction reaches while the other one is busy,
 * the ceiling for concurrent save and load. The rate of two concurrent copies depends on which
 * streams carry them (streams share a few hardware queues), so four pairs out of four new
 * streams are measured, `repeats` copies each way per pair, and the pair with the highest sum
 * is reported. Allocates 2 x bytes of pinned and of device memory. */
int kvt_measure_pcie_both_ways(int device, uint64_t bytes, uint32_t repeats, double* d2h_bytes_per_s,
                               double* h2d_bytes_per_s);

/* ---------------------------------------- store objects found by block hash */

/* A ring of store objects in pinned host memory, found by key (the block hash): the staging
 * tier between the paged cache and a KV store. Mirrors what FileBackend does with a block
 *                                  blade_kvt/hybrid_connector/file_backend.py:215-285
 * (a block whose hash is stored already is skipped on save, _blk_ready(); a load finds the
 * block by its hash), with one entry per block holding that block of ALL layers, i.e. one
 * object of kvt_plan_create_objects with object_stride = entry_bytes. Entries are handed out in
 * ring order, so the new blocks of a batch are neighbours and cross PCIe as one or two large
 * DMA copies; when the ring is full the oldest entries are given to new keys.
 * device = KVT_DEVICE_NONE gives an index over plain host memory (no save / load), for a store
 * that fills the entries itself. Keys are key_bytes (1..256) each, compared byte for byte.
 * Calls may come from several threads: an entry whose bytes a caller was asked for stays with
 * its key until that caller has written it (save / commit) or given up (release), so EVERY
 * is_new answer must be followed by exactly one of the three (an answer that is never settled
 * keeps its entry out of circulation); a load can name the keys it expects. */
typedef struct kvt_object_ring kvt_object_ring;
int kvt_object_ring_create(int device, uint64_t entry_bytes, uint32_t n_entries,
                           uint32_t key_bytes, kvt_object_ring** out);
void kvt_object_ring_destroy(kvt_object_ring* r);
/* Host address of an entry (for the store behind the ring: file or network IO). */
void* kvt_object_ring_entry(kvt_object_ring* r, uint32_t entry);
/* Save side. For each of the n keys: entries[i] = its entry; is_new[i] = 1 when the caller has
 * to provide the block's bytes (a fresh entry was assigned, or an earlier reservation was never
 * written), 0 when the block is stored already or appeared earlier in this call. No entry that
 * this call refers to is given away by it, nor one that some caller has yet to write;
 * KVT_ERR_INVALID (nothing reserved) when the batch has more new blocks than the entries that
 * are left. An entry given to a new key is waited for first if a transfer still uses it. */
int kvt_object_ring_reserve(kvt_object_ring* r, const void* keys, uint32_t n, uint32_t* entries,
                            uint8_t* is_new);
/* Device -> entries: object i (entry_bytes long) at dev + i * dev_stride goes to entries[i];
 * neighbouring entries whose objects are neighbours too (dev_stride == entry_bytes) are one
 * copy. Ordered behind the work queued on `stream` (the pack that produces the objects);
 * `stream` continues once the objects have left the buffer. The entries count as written from
 * here on (kvt_object_ring_wait before the HOST reads one). */
int kvt_object_ring_save(kvt_object_ring* r, const uint32_t* entries, uint32_t n, const void* dev,
                         uint64_t dev_stride, void* stream);
/* Marks entries as written that the caller filled through kvt_object_ring_entry. */
int kvt_object_ring_commit(kvt_object_ring* r, const uint32_t* entries, uint32_t n);
/* Gives up being asked for these entries' bytes (a failed batch). When nobody else was asked
 * for the same block and it has not been written, its key is forgotten and the entry may be
 * given away again. */
int kvt_object_ring_release(kvt_object_ring* r, const uint32_t* entries, uint32_t n);
/* Load side: found[i] = 1 and entries[i] when key i is stored (written or its write queued). */
int kvt_object_ring_lookup(kvt_object_ring* r, const void* keys, uint32_t n, uint32_t* entries,
                           uint8_t* found);
/* Entries -> device, the mirror of save; work queued on `stream` afterwards (the unpack) sees
 * the objects. keys (may be NULL): the n keys the lookup was made with; when another thread's
 * reserve has given one of the entries to a different block meanwhile, nothing is copied and
 * KVT_ERR_OUT_OF_RANGE says so (look up again). */
int kvt_object_ring_load(kvt_object_ring* r, const uint32_t* entries, const void* keys, uint32_t n,
                         void* dev, uint64_t dev_stride, void* stream);
/* Host-blocking: the last save / load that touches the entry has completed. */
int kvt_object_ring_wait(kvt_object_ring* r, uint32_t entry);
/* Counters since creation (what a store reports as its hit rate and traffic). */
typedef struct kvt_object_ring_counters {
  uint64_t blocks_asked_for;      /* is_new answers of reserve                                   */
  uint64_t blocks_already_here;   /* the other answers: stored, or repeated inside a batch       */
  uint64_t entries_given_away;    /* stored or reserved keys dropped to make room                */
  uint64_t lookups_found, lookups_missed;
  uint64_t bytes_saved, bytes_loaded;   /* through kvt_object_ring_save / _load                  */
  uint64_t entries_in_use;        /* keys in the index now                                       */
} kvt_object_ring_counters;
int kvt_object_ring_stats(kvt_object_ring* r, kvt_object_ring_counters* out);

/* ------------------------------------------------------------- utilities */

/* Plain device-to-device copy kernel with the same vector width and launch
 * shape as the gather kernel; used to calibrate profiler counters and as the
 * "no scatter" bandwidth reference. */
int kvt_copy_linear(void* dst, const void* src, uint64_t bytes, void* stream);
/* The HIP runtime's own device-to-device copy (hipMemcpyAsync) of the same bytes: a copy rate
 * of the part that owes nothing to this library's kernels, timed beside them. */
int kvt_copy_runtime_d2d(void* dst, const void* src, uint64_t bytes, void* stream);
/* Average duration in milliseconds of the GPU work queued on `stream` between
 * two internally created events around `fn`-less region helpers: */
int kvt_event_create(void** ev);
int kvt_event_destroy(void* ev);
int kvt_event_record(void* ev, void* stream);
int kvt_event_synchronize(void* ev);
int kvt_event_elapsed_ms(void* start, void* stop, float* ms);
int kvt_stream_create(void** stream);
int kvt_stream_destroy(void* stream);
int kvt_stream_synchronize(void* stream);

#ifdef __cplusplus
}
#endif
#endif  /* KVT_HIP_H_ */
