// ep::CudaStream over a HIP stream: the device stream OneFlow's user kernels receive through
// KernelComputeContext::stream() (oneflow/core/ep/include/stream.h:30-57) with the members of
// oneflow/core/ep/cuda/cuda_stream.h:73-118 that the quantized-inference kernels and the runtime
// around them use: cuda_stream(), Sync, RecordEvent, WaitEvent, GetAsyncError,
// OnExecutionContextSetup / Teardown and the launch-size helper over the CU count.  Class and
// member names keep the reference's spelling so that kernel sources (`ctx->stream()
// ->As<ep::CudaStream>()->cuda_stream()`) are one text for both builds; on this device the handle
// is a hipStream_t.  Written against the C ABI of ofq_hip_shim.h: no HIP header is included.
//
// Left out on purpose (other layers of the reference, not reached by these kernels): the
// cuBLAS / cuDNN / cuSOLVER handles and their workspace, stream-ordered allocation
// (AllocAsync / FreeAsync stay at ep::Stream's default "unimplemented"), the CUDA-graph capture
// helpers, and CudaDevice (device() is replaced by device_index()).
#pragma once

#include <algorithm>
#include <cstddef>
#include <cstdint>

#include "oneflow/core/ep/include/stream.h"
#include "oneflow/core/ep/cuda/cuda_event.h"

namespace oneflow {
namespace ep {

using cudaStream_t = void*;

struct CudaLaunchConfig {
  uint32_t grid_dim;
  uint32_t block_dim;
  size_t shared_mem_size;
  CudaLaunchConfig() : grid_dim(0), block_dim(0), shared_mem_size(0) {}
  CudaLaunchConfig(uint32_t grid_size, uint32_t block_size, size_t shared_mem_size)
      : grid_dim(grid_size), block_dim(block_size), shared_mem_size(shared_mem_size) {}
};

class CudaStream : public Stream {
 public:
  CudaStream(const CudaStream&) = delete;
  CudaStream& operator=(const CudaStream&) = delete;
  // a stream of its own on `device_index` (default priority), synchronised and destroyed with
  // the object
  explicit CudaStream(int device_index);
  // a view of a stream somebody else owns (a framework's current stream): never destroyed here
  CudaStream(int device_index, cudaStream_t borrowed);
  ~CudaStream() override;

  static constexpr uint32_t kDefaultBlockSize = 256;

  DeviceType device_type() const override;
  int device_index() const { return device_index_; }
  Maybe<void> Sync() override;
  void RecordEvent(Event* event) override;
  void WaitEvent(Event* event) override;
  Maybe<void> GetAsyncError() override;

  Maybe<void> OnExecutionContextSetup() override;
  Maybe<void> OnExecutionContextTeardown() override;

  cudaStream_t cuda_stream() const { return cuda_stream_; }

  // device_properties().multiProcessorCount / .maxThreadsPerMultiProcessor of the reference
  int multi_processor_count() const { return cu_count_; }
  int max_threads_per_multi_processor() const { return max_threads_per_cu_; }

  void InitLaunchConfigWithWaves(CudaLaunchConfig* config, size_t elem_cnt, size_t block_size,
                                 size_t max_waves) const {
    const uint32_t max_grid_size =
        (uint32_t)(max_waves * (size_t)cu_count_ * ((size_t)max_threads_per_cu_ / block_size));
    const uint32_t grid_size =
        std::min<uint32_t>(max_grid_size, (uint32_t)((elem_cnt + block_size - 1) / block_size));
    config->grid_dim = grid_size;
    config->block_dim = (uint32_t)block_size;
    config->shared_mem_size = 0;
  }

 private:
  void QueryDevice();
  int device_index_;
  cudaStream_t cuda_stream_;
  bool owned_;
  int cu_count_ = 0;
  int max_threads_per_cu_ = 0;
};

}  // namespace ep
}  // namespace oneflow
