// ep::CudaEvent over a HIP event: the class OneFlow's stream layer records and waits on
// (oneflow/core/ep/cuda/cuda_event.h:28-43, cuda_event.cpp), written against the C ABI of
// ofq_hip_shim.h so that no HIP header is needed here.  The handle type keeps the reference's
// spelling; on this device it is a hipEvent_t.
#pragma once

#include "oneflow/core/ep/include/event.h"

namespace oneflow {
namespace ep {

using cudaEvent_t = void*;

class CudaEvent : public Event {
 public:
  CudaEvent(const CudaEvent&) = delete;
  CudaEvent& operator=(const CudaEvent&) = delete;
  // flags: kept for the reference's signature; events are created without timing, which is what
  // the reference's stream layer asks for (cudaEventDisableTiming)
  explicit CudaEvent(unsigned int flags);
  ~CudaEvent() override;

  Maybe<bool> QueryDone() override;
  Maybe<void> Sync() override;

  cudaEvent_t cuda_event();

 private:
  cudaEvent_t cuda_event_;
};

}  // namespace ep
}  // namespace oneflow
