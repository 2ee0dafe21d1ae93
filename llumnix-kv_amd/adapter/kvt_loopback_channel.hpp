// An IChannel (kvtransfer/include/channel.h:59-83) whose "wire" is a transfer
// buffer in HBM: send_data(layer) packs the layer out of the sender's paged cache
// on the library's side stream and unpacks it into the receiver's paged cache on
// the same GPU. It is what TCPChannel + TCPServer do to the bytes
// (kvtransfer/src/tcp_channel.cpp:348-475 register_data, :517-560 send_data,
// :190-261 handle_kv_cache_data) with the network taken out, and plugs in where
// the reference's own tests plug FakeChannel (kvtransfer/tests/send_stub_test.cpp:173-209):
// behind an IChannelFactory handed to KvSendStub.
//
// Like kvt_blade_adapter.hpp this header is compiled INSIDE the Blade-KVT tree.
//
// Protocol kept from the reference:
//   * register_data borrows `data` until flush(); with TPKind::PEQD every tensor's
//     list is merged IN PLACE (sorted by source offset, touching ranges joined,
//     emptied entries erased) exactly as TCPChannel::register_data leaves it;
//     other kinds are sent as they are and must hold a single tensor;
//   * the receiver validates the destination offsets before it scatters
//     (validate_ipc_block_bounds, kvtransfer/src/channel.cpp:11-50) and throws
//     std::out_of_range on a bad range;
//   * send_data may return before the bytes have moved; flush() blocks until every
//     layer sent so far has landed and writes the reference's metric keys
//     (OriginSbNum, MergedSbNum, SbSizeMin, SbSizeMax, SbSizeTotal) as `k=v,`.
// Layer readiness: send_data(layer) never blocks the host. The pack is ordered
// after the work already queued on `compute_stream` (the stream the engine writes
// the layer's KV on) by an event, where the reference parks a host thread in
// cudaEventSynchronize (Step::wait_layer_ready, kvtransfer/src/step.cpp:49-69).
#ifndef KVT_LOOPBACK_CHANNEL_HPP_
#define KVT_LOOPBACK_CHANNEL_HPP_

#include <algorithm>
#include <limits>
#include <sstream>
#include <string>
#include <vector>

#include "kvt_blade_adapter.hpp"

namespace kvt_adapter {

class LoopbackChannel : public blade_llm::IChannel {
 public:
  // src_layers / dst_layers: device base pointers, [layer * n_tensors + tensor];
  // *_capacity: bytes of tensor t of one layer (block_sizes[t] * layer_num_blocks).
  // alloc / release provide the transfer buffer (device memory), e.g. hipMalloc / hipFree
  // or a framework's allocator.
  LoopbackChannel(int device, std::vector<void*> src_layers, std::vector<uint64_t> src_capacity,
                  std::vector<void*> dst_layers, std::vector<uint64_t> dst_capacity,
                  uint32_t n_layers, void* compute_stream, void* (*alloc)(size_t),
                  void (*release)(void*))
      : device_(device), src_cap_(std::move(src_capacity)), dst_cap_(std::move(dst_capacity)),
        n_layers_(n_layers), compute_(compute_stream), alloc_(alloc), release_(release) {
    const uint32_t n_tensors = static_cast<uint32_t>(src_cap_.size());
    if (n_tensors == 0 || dst_cap_.size() != n_tensors || n_layers == 0 ||
        src_layers.size() != static_cast<size_t>(n_layers) * n_tensors ||
        dst_layers.size() != src_layers.size())
      throw std::runtime_error("LoopbackChannel: layer pointer tables do not match the tensor count");
    raise(kvt_cache_register(device, src_layers.data(), n_layers, n_tensors, src_cap_.data(), &src_));
    const int rc = kvt_cache_register(device, dst_layers.data(), n_layers, n_tensors,
                                      dst_cap_.data(), &dst_);
    if (rc != KVT_OK) {
      kvt_cache_destroy(src_);
      raise(rc);
    }
  }

  ~LoopbackChannel() override {
    active_ = false;
    drop_batch();
    kvt_cache_destroy(src_);
    kvt_cache_destroy(dst_);
  }

  LoopbackChannel(const LoopbackChannel&) = delete;
  LoopbackChannel& operator=(const LoopbackChannel&) = delete;

  void connect(const blade_llm::WorkerInfo& dst_info) override {
    dst_inst_id_ = dst_info.inst_id;
    dst_worker_id_ = dst_info.worker_id;
    active_ = true;
  }

  void register_data(std::vector<std::vector<blade_llm::IpcBlock>>& data,
                     blade_llm::TPKind kind) override {
    if (!active_) throw std::runtime_error("LoopbackChannel: register_data before connect");
    if (session_) throw std::runtime_error("LoopbackChannel: register_data twice without flush");
    if (data.size() != src_cap_.size())
      throw std::runtime_error("LoopbackChannel: data does not hold one list per cache tensor");
    origin_ = merged_ = total_ = 0;
    min_ = std::numeric_limits<size_t>::max();
    max_ = 0;
    if (kind == blade_llm::TPKind::PEQD) {
      for (auto& tensor_data : data) {
        origin_ += tensor_data.size();
        const auto [mn, mx, tot, cnt] = kvt_adapter::merge_interval(tensor_data);  // sorts, joins, erases
        merged_ += cnt;
        if (cnt) min_ = std::min(min_, mn);
        max_ = std::max(max_, mx);
        total_ += tot;
      }
    } else {
      if (data.size() != 1)
        throw std::runtime_error("LoopbackChannel: a TP-remapping batch holds a single tensor");
      origin_ = merged_ = data[0].size();
      for (const auto& b : data[0]) {
        min_ = std::min(min_, b.length);
        max_ = std::max(max_, b.length);
        total_ += b.length;
      }
    }
    if (merged_ == 0) min_ = 0;
    // receiver side: refuse metadata that would scatter outside the registered cache
    for (size_t t = 0; t < data.size(); ++t)
      kvt_adapter::validate_ipc_block_bounds(data[t], dst_cap_[t],
                                             blade_llm::IpcBlockOffset::DESTINATION);
    try {
      build(data, kind);
    } catch (...) {
      drop_batch();
      throw;
    }
  }

  void send_data(size_t layer_index) override {
    if (!session_) throw std::runtime_error("LoopbackChannel: send_data without register_data");
    if (layer_index >= n_layers_) throw std::out_of_range("LoopbackChannel: layer index");
    const uint32_t layer = static_cast<uint32_t>(layer_index);
    raise(kvt_session_save_layer(session_, layer, compute_));
    // the scatter follows the gather on the same side stream
    raise(kvt_unpack(plan_, dst_, layer, 1, static_cast<uint8_t*>(packed_) + layer * stride_,
                     stride_, kvt_session_side_stream(session_)));
    ++sent_;
  }

  void flush(std::string& out) override {
    std::ostringstream os;
    os << "OriginSbNum=" << origin_ << ",MergedSbNum=" << merged_ << ",SbSizeMin=" << min_
       << ",SbSizeMax=" << max_ << ",SbSizeTotal=" << total_ << ",LayersSent=" << sent_ << ",";
    out = os.str();
    if (session_) {
      const int rc = kvt_stream_synchronize(kvt_session_side_stream(session_));
      drop_batch();
      raise(rc);
    }
  }

  bool is_active() override { return active_; }

  void close() override {
    active_ = false;
    drop_batch();  // releases the transfer buffer as well
  }

 private:
  void build(std::vector<std::vector<blade_llm::IpcBlock>>& data, blade_llm::TPKind kind) {
    kvt_block_lists* lists = nullptr;
    raise(kvt_block_lists_create(&lists));
    int rc = KVT_OK;
    for (size_t t = 0; t < data.size() && rc == KVT_OK; ++t)
      rc = kvt_block_lists_append(lists, static_cast<uint32_t>(t),
                                  reinterpret_cast<const kvt_ipc_block*>(data[t].data()),
                                  data[t].size());
    if (rc == KVT_OK && kind != blade_llm::TPKind::PEQD) {
      // one short range per token: hand the kernel (base, stride) records instead
      kvt_run_lists* runs = nullptr;
      rc = kvt_run_lists_create(&runs);
      if (rc == KVT_OK) rc = kvt_run_lists_compress(lists, runs);
      if (rc == KVT_OK)
        rc = kvt_plan_create_runs(device_, runs, src_cap_.data(), dst_cap_.data(), 0, &plan_);
      kvt_run_lists_destroy(runs);
    } else if (rc == KVT_OK) {
      rc = kvt_plan_create(device_, lists, src_cap_.data(), dst_cap_.data(), nullptr, 0, &plan_);
    }
    kvt_block_lists_destroy(lists);
    raise(rc);
    stride_ = kvt_plan_layer_bytes(plan_);
    const size_t need = static_cast<size_t>(std::max<uint64_t>(stride_, 256)) * n_layers_;
    if (need > packed_bytes_) {
      if (packed_) release_(packed_);
      packed_ = alloc_(need);
      packed_bytes_ = packed_ ? need : 0;
      if (!packed_) throw std::runtime_error("LoopbackChannel: transfer buffer allocation failed");
    }
    raise(kvt_session_create(plan_, src_, packed_, stride_, &session_));
    sent_ = 0;
  }

  // ends the current batch; an active channel keeps its transfer buffer for the next one
  void drop_batch() {
    if (session_) kvt_session_destroy(session_);  // waits for the side stream
    session_ = nullptr;
    if (plan_) kvt_plan_destroy(plan_);
    plan_ = nullptr;
    if (!active_ && packed_) {
      release_(packed_);
      packed_ = nullptr;
      packed_bytes_ = 0;
    }
  }

  int device_;
  std::vector<uint64_t> src_cap_, dst_cap_;
  uint32_t n_layers_;
  void* compute_;
  void* (*alloc_)(size_t);
  void (*release_)(void*);
  kvt_cache* src_ = nullptr;
  kvt_cache* dst_ = nullptr;
  kvt_plan* plan_ = nullptr;
  kvt_session* session_ = nullptr;
  void* packed_ = nullptr;
  size_t packed_bytes_ = 0;
  uint64_t stride_ = 0;
  size_t origin_ = 0, merged_ = 0, min_ = 0, max_ = 0, total_ = 0, sent_ = 0;
  bool active_ = false;
  blade_llm::InstanceId dst_inst_id_;
  blade_llm::WorkerId dst_worker_id_ = 0;
};

}  // namespace kvt_adapter

#endif  // KVT_LOOPBACK_CHANNEL_HPP_
