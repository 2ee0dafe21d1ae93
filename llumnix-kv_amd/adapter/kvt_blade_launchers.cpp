// Link-level stand-in for the reference's kernel file: the four extern "C"
// launchers that kvtransfer/src/copy_kernels.cpp declares (:52-85, :101-108) and
// kvtransfer/src/copy_kernels.cu defines (:93-103, :179-192, :268-281, :467-481),
// with the same names, argument order and meaning, forwarding to libkvt_hip.so.
// Built into a Blade-KVT tree INSTEAD of copy_kernels.cu, the host policy code in
// copy_kernels.cpp (batching, metadata upload, method selection) keeps working
// unchanged on an MI355X; the stream argument is a hipStream_t there.
//
// num_cuda_blocks / threads_per_block are the reference's persistent grid (resident blocks per
// SM x SMs x BLLM_KVTRANS_KERNEL_COPY_SM_USAGE, copy_kernels.cpp:327-335), sized for another
// machine: they are not passed on. The library picks its own launch shape, and the share of
// the device is set once with kvt_set_copy_cu_usage (kvt_adapter::apply_kernel_copy_sm_usage
// reads the same variable).
//
// The reference's launchers return nothing and cannot report a failed launch;
// here a refused call (null argument, no device) is written to stderr.
#include <cstdint>
#include <cstdio>

#include "kvt_hip.h"

namespace {
void report(int rc, const char* who) {
  if (rc != KVT_OK) std::fprintf(stderr, "%s: %s\n", who, kvt_last_error());
}
}  // namespace

extern "C" {

void launch_copy_int64_array_h2d_kernel(const int64_t* host_src, int64_t* device_dst,
                                        int64_t num_elements, int num_cuda_blocks,
                                        int threads_per_block, void* stream) {
  (void)num_cuda_blocks;
  (void)threads_per_block;
  report(kvt_launch_copy_int64_array_h2d(host_src, device_dst, num_elements, 0, 0, stream),
         "launch_copy_int64_array_h2d_kernel");
}

void launch_copy_h2d_direct_kernel(const char* host_src, char* gpu_dst_base,
                                   const int64_t* src_offsets, const int64_t* dst_offsets,
                                   const int64_t* lengths, int64_t num_blocks, int num_cuda_blocks,
                                   int threads_per_block, void* stream) {
  (void)num_cuda_blocks;
  (void)threads_per_block;
  report(kvt_launch_copy_h2d_direct(host_src, gpu_dst_base, src_offsets, dst_offsets, lengths,
                                    num_blocks, 0, 0, stream),
         "launch_copy_h2d_direct_kernel");
}

void launch_copy_d2h_direct_kernel(const char* gpu_src_base, char* host_dst,
                                   const int64_t* src_offsets, const int64_t* dst_offsets,
                                   const int64_t* lengths, int64_t num_blocks, int num_cuda_blocks,
                                   int threads_per_block, void* stream) {
  (void)num_cuda_blocks;
  (void)threads_per_block;
  report(kvt_launch_copy_d2h_direct(gpu_src_base, host_dst, src_offsets, dst_offsets, lengths,
                                    num_blocks, 0, 0, stream),
         "launch_copy_d2h_direct_kernel");
}

void launch_copy_d2h_bf16_to_fp8_kernel(const char* gpu_src_base, void* host_dst,
                                        const int64_t* src_offsets, const int64_t* dst_offsets,
                                        const int64_t* lengths, int64_t num_blocks,
                                        int num_cuda_blocks, int threads_per_block, void* stream) {
  (void)num_cuda_blocks;
  (void)threads_per_block;
  report(kvt_launch_copy_d2h_bf16_to_fp8(gpu_src_base, host_dst, src_offsets, dst_offsets, lengths,
                                         num_blocks, 0, 0, stream),
         "launch_copy_d2h_bf16_to_fp8_kernel");
}

}  // extern "C"
