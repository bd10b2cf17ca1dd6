// Stand-alone build only: the slice of oneflow/core/ep/cuda/cuda_stream.h the adapter uses.
// ep::CudaStream hands out the raw device stream (cuda_stream(), reference line 91); on a ROCm
// build of the EP layer that handle is the hipStream_t.  Same include path and same spelling as
// in a OneFlow tree, so the adapter source is one text for both builds.
#pragma once

#include "oneflow/core/framework/framework.h"

namespace oneflow {
namespace ep {

using cudaStream_t = void*;

class CudaStream final : public Stream {
 public:
  explicit CudaStream(cudaStream_t s) : stream_(s) {}
  cudaStream_t cuda_stream() const { return stream_; }

 private:
  cudaStream_t stream_;
};

}  // namespace ep
}  // namespace oneflow
