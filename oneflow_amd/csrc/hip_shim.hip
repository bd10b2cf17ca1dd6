// The HIP runtime calls behind ofq_hip_shim.h: device selection, streams, events and the
// asynchronous-error query that OneFlow's ep::CudaStream / ep::CudaEvent need.
#include <hip/hip_runtime.h>

#include "ofq_device.h"
#include "ofq_hip_shim.h"

namespace ofq {
namespace {
// the launch error an entry point of this library consumed while reporting OFQ_ERR_LAUNCH
thread_local int pending_launch_error = 0;
}  // namespace

void note_launch_error(int hip_error) {
  if (pending_launch_error == 0) pending_launch_error = hip_error;
}
}  // namespace ofq

extern "C" const char* ofq_hip_error_string(int hip_error) {
  return hipGetErrorString(static_cast<hipError_t>(hip_error));
}

extern "C" int ofq_hip_device_count(int* count) { return (int)hipGetDeviceCount(count); }
extern "C" int ofq_hip_set_device(int device) { return (int)hipSetDevice(device); }
extern "C" int ofq_hip_get_device(int* device) { return (int)hipGetDevice(device); }

extern "C" int ofq_hip_device_cu_count(int device, int* cu_count) {
  return (int)hipDeviceGetAttribute(cu_count, hipDeviceAttributeMultiprocessorCount, device);
}
extern "C" int ofq_hip_device_max_threads_per_cu(int device, int* threads) {
  return (int)hipDeviceGetAttribute(threads, hipDeviceAttributeMaxThreadsPerMultiProcessor, device);
}

extern "C" int ofq_hip_stream_create(int device, void** stream) {
  if (stream == nullptr) return (int)hipErrorInvalidValue;
  int prev = -1;
  hipError_t e = hipGetDevice(&prev);
  if (e != hipSuccess) return (int)e;
  if (prev != device && (e = hipSetDevice(device)) != hipSuccess) return (int)e;
  hipStream_t s = nullptr;
  e = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);  // default priority
  if (prev != device) (void)hipSetDevice(prev);
  *stream = s;
  return (int)e;
}
extern "C" int ofq_hip_stream_destroy(void* stream) {
  return (int)hipStreamDestroy(static_cast<hipStream_t>(stream));
}
extern "C" int ofq_hip_stream_synchronize(void* stream) {
  return (int)hipStreamSynchronize(static_cast<hipStream_t>(stream));
}

extern "C" int ofq_hip_event_create(void** event) {
  if (event == nullptr) return (int)hipErrorInvalidValue;
  hipEvent_t ev = nullptr;
  const hipError_t e = hipEventCreateWithFlags(&ev, hipEventDisableTiming);
  *event = ev;
  return (int)e;
}
extern "C" int ofq_hip_event_destroy(void* event) {
  return (int)hipEventDestroy(static_cast<hipEvent_t>(event));
}
extern "C" int ofq_hip_event_record(void* event, void* stream) {
  return (int)hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream));
}
extern "C" int ofq_hip_stream_wait_event(void* stream, void* event) {
  return (int)hipStreamWaitEvent(static_cast<hipStream_t>(stream), static_cast<hipEvent_t>(event), 0);
}
extern "C" int ofq_hip_event_query(void* event, int* done) {
  const hipError_t e = hipEventQuery(static_cast<hipEvent_t>(event));
  if (e == hipSuccess || e == hipErrorNotReady) {
    if (done != nullptr) *done = e == hipSuccess ? 1 : 0;
    return 0;
  }
  return (int)e;
}
extern "C" int ofq_hip_event_synchronize(void* event) {
  return (int)hipEventSynchronize(static_cast<hipEvent_t>(event));
}

extern "C" int ofq_hip_get_async_error(void) {
  const int kept = ofq::pending_launch_error;
  ofq::pending_launch_error = 0;
  const hipError_t now = hipGetLastError();  // clears the runtime's own record
  return kept != 0 ? kept : (int)now;
}
