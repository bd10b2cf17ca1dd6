// ep::CudaStream and ep::CudaEvent on a HIP device (see cuda_stream.h); the device runtime is
// reached through ofq_hip_shim.h only.
#include "oneflow/core/ep/cuda/cuda_stream.h"

#include "ofq_hip_shim.h"

namespace oneflow {
namespace ep {

namespace {

// the reference's OF_CUDA_CHECK: an error of the device runtime outside a Maybe-returning
// function ends the process with the runtime's message
void CheckHip(int err, const char* what) {
  if (err != 0) {
    std::cerr << what << ": " << ofq_hip_error_string(err) << " (" << err << ")\n";
    CHECK_EQ(err, 0);
  }
}

Maybe<void> ToMaybe(int err) {
  if (err == 0) { return Maybe<void>::Ok(); }
  return Error::RuntimeError() << ofq_hip_error_string(err) << " (" << err << ") ";
}

}  // namespace

// ---- CudaEvent (cuda_event.cpp) ---------------------------------------------------------------
CudaEvent::CudaEvent(unsigned int /*flags*/) : cuda_event_(nullptr) {
  CheckHip(ofq_hip_event_create(&cuda_event_), "hipEventCreateWithFlags");
}

CudaEvent::~CudaEvent() { CheckHip(ofq_hip_event_destroy(cuda_event_), "hipEventDestroy"); }

Maybe<bool> CudaEvent::QueryDone() {
  int done = 0;
  const int err = ofq_hip_event_query(cuda_event_, &done);
  if (err != 0) {
    return Error::RuntimeError() << ofq_hip_error_string(err) << " (" << err << ") ";
  }
  return done != 0;
}

Maybe<void> CudaEvent::Sync() { return ToMaybe(ofq_hip_event_synchronize(cuda_event_)); }

cudaEvent_t CudaEvent::cuda_event() { return cuda_event_; }

// ---- CudaStream (cuda_stream.cpp:95-103,195-247) ----------------------------------------------
CudaStream::CudaStream(int device_index)
    : device_index_(device_index), cuda_stream_(nullptr), owned_(true) {
  CheckHip(ofq_hip_stream_create(device_index_, &cuda_stream_), "hipStreamCreateWithFlags");
  QueryDevice();
}

CudaStream::CudaStream(int device_index, cudaStream_t borrowed)
    : device_index_(device_index), cuda_stream_(borrowed), owned_(false) {
  QueryDevice();
}

CudaStream::~CudaStream() {
  if (owned_) {
    CheckHip(ofq_hip_stream_synchronize(cuda_stream_), "hipStreamSynchronize");
    CheckHip(ofq_hip_stream_destroy(cuda_stream_), "hipStreamDestroy");
  }
}

void CudaStream::QueryDevice() {
  CheckHip(ofq_hip_device_cu_count(device_index_, &cu_count_), "hipDeviceGetAttribute");
  CheckHip(ofq_hip_device_max_threads_per_cu(device_index_, &max_threads_per_cu_),
           "hipDeviceGetAttribute");
}

Maybe<void> CudaStream::OnExecutionContextSetup() {
  return ToMaybe(ofq_hip_set_device(device_index_));
}

Maybe<void> CudaStream::OnExecutionContextTeardown() { return Maybe<void>::Ok(); }

DeviceType CudaStream::device_type() const { return DeviceType::kCUDA; }

Maybe<void> CudaStream::Sync() { return ToMaybe(ofq_hip_stream_synchronize(cuda_stream_)); }

void CudaStream::RecordEvent(Event* event) {
  auto* cuda_event = static_cast<CudaEvent*>(event);  // NOLINT
  CheckHip(ofq_hip_event_record(cuda_event->cuda_event(), cuda_stream_), "hipEventRecord");
}

void CudaStream::WaitEvent(Event* event) {
  auto* cuda_event = static_cast<CudaEvent*>(event);  // NOLINT
  CheckHip(ofq_hip_stream_wait_event(cuda_stream_, cuda_event->cuda_event()),
           "hipStreamWaitEvent");
}

Maybe<void> CudaStream::GetAsyncError() { return ToMaybe(ofq_hip_get_async_error()); }

}  // namespace ep
}  // namespace oneflow
