/*
 * The HIP device / stream layer behind OneFlow's execution-provider stream, as a C ABI.
 *
 * OneFlow's user kernels reach the device through ep::Stream
 *   (oneflow/core/ep/include/stream.h:30-57) and its CUDA implementation ep::CudaStream
 *   (oneflow/core/ep/cuda/cuda_stream.h:73-91, cuda_stream.cpp:209-247) and ep::CudaEvent
 *   (oneflow/core/ep/cuda/cuda_event.h:28-43).
 * The functions below are what those classes need from the device runtime on an MI355X: the
 * C++ classes of the same names in oneflow_amd/plugin/ep_hip/ are written against this header
 * only, so the host side of the kernel layer compiles with a plain C++ compiler and never
 * includes a HIP header.  Streams are created at the default priority.
 *
 * Every function returns 0 on success and the hipError_t value otherwise
 * (ofq_hip_error_string() names it); nothing here allocates device memory.
 */
#ifndef OFQ_HIP_SHIM_H_
#define OFQ_HIP_SHIM_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* ofq_hip_error_string(int hip_error);

/* device: CudaStream::OnExecutionContextSetup = cudaSetDevice (cuda_stream.cpp:209-213);
 * device_properties().multiProcessorCount (cuda_stream.h:111,117-118) = the CU count */
int ofq_hip_device_count(int* count);
int ofq_hip_set_device(int device);
int ofq_hip_get_device(int* device);
int ofq_hip_device_cu_count(int device, int* cu_count);
int ofq_hip_device_max_threads_per_cu(int device, int* threads);

/* stream: CudaStream::CudaStream / ~CudaStream / Sync (cuda_stream.cpp:95-103,195-207,221-228) */
int ofq_hip_stream_create(int device, void** stream);
int ofq_hip_stream_destroy(void* stream);
int ofq_hip_stream_synchronize(void* stream);

/* events: CudaEvent (cuda_event.cpp), CudaStream::RecordEvent / WaitEvent
 * (cuda_stream.cpp:230-238).  query: *done = 1 when the event has completed, 0 while pending */
int ofq_hip_event_create(void** event);
int ofq_hip_event_destroy(void* event);
int ofq_hip_event_record(void* event, void* stream);
int ofq_hip_stream_wait_event(void* stream, void* event);
int ofq_hip_event_query(void* event, int* done);
int ofq_hip_event_synchronize(void* event);

/* CudaStream::GetAsyncError = cudaGetLastError (cuda_stream.cpp:240-247): the error left by the
 * last launch of the calling thread and cleared by this call.  A launch that one of this
 * library's entry points reported as OFQ_ERR_LAUNCH is kept for this call as well (the entry
 * point has to read the runtime's error to report it), so the runtime's check after Compute
 * (oneflow/user/kernels/stateful_opkernel.cpp:1007) sees it either way. */
int ofq_hip_get_async_error(void);

#ifdef __cplusplus
}
#endif
#endif /* OFQ_HIP_SHIM_H_ */
