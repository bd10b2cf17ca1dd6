// Stand-alone build only: the slice of oneflow/core/kernel/cuda_graph_support.h the adapter
// uses (a kernel derives user_op::CudaGraphSupport to declare that its Compute may run under
// stream capture, reference lines 29-41).
#pragma once

namespace oneflow {
namespace user_op {

class KernelInitContext;
class KernelComputeContext;
class OpKernelState;
class OpKernelCache;

class CudaGraphSupport {
 public:
  CudaGraphSupport() = default;
  virtual ~CudaGraphSupport() = default;
  virtual bool IsCudaGraphSupported(KernelInitContext*, OpKernelState*) const { return true; }
  virtual bool IsReadyForCapture(KernelComputeContext*, OpKernelState*, const OpKernelCache*) const {
    return true;
  }
};

}  // namespace user_op
}  // namespace oneflow
