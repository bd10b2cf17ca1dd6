// Measurement probes of the benchmark (bench_probes.h): a kernel that only reads, an empty
// kernel, a plain copy.  Built into libofq_bench_probes.so, not into the product library.
#include "bench_probes.h"
#include "ofq_device.h"

namespace ofq {
// (the product library defines this in hip_shim.hip; this library stands alone)
void note_launch_error(int) {}

namespace {

// One 16-byte request per lane, the whole buffer in one round, nothing computed beyond a value
// that keeps the loads alive: the time below which no kernel that has to read those bytes once
// can finish.
__global__ void __launch_bounds__(256)
probe_read_kernel(const u32x4* __restrict__ p, size_t nvec, uint32_t* sink) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const u32x4 v = __builtin_nontemporal_load(p + (i < nvec ? i : nvec - 1));
  const uint32_t a = v[0] ^ v[1] ^ v[2] ^ v[3];
  if (a == 0x9E3779B9u && sink != nullptr) sink[0] = a;  // practically never: keeps the load
}

__global__ void __launch_bounds__(256) empty_kernel(uint32_t* sink) {
  if (threadIdx.x == 0xFFFFu) sink[0] = 1u;  // never
}

__global__ void __launch_bounds__(256)
copy_kernel(u32x4* __restrict__ dst, const u32x4* __restrict__ src, size_t nvec) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < nvec) dst[i] = src[i];
}

}  // namespace
}  // namespace ofq

extern "C" int ofq_bench_probe_read(void* stream, const void* buf, size_t bytes, void* sink) {
  if (buf == nullptr || sink == nullptr) return OFQ_ERR_NULL_POINTER;
  if ((reinterpret_cast<uintptr_t>(buf) & 15) != 0) return OFQ_ERR_MISALIGNED;
  if (bytes < 16) return OFQ_ERR_BAD_SHAPE;
  const size_t nvec = bytes / 16;
  const size_t blocks = (nvec + 255) / 256;
  if (blocks > 0x7FFFFFFFull) return OFQ_ERR_BAD_SHAPE;
  ofq::probe_read_kernel<<<(unsigned)blocks, 256, 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const ofq::u32x4*>(buf), nvec, static_cast<uint32_t*>(sink));
  return ofq_check_launch();
}

extern "C" int ofq_bench_empty_launch(void* stream, void* sink) {
  if (sink == nullptr) return OFQ_ERR_NULL_POINTER;
  ofq::empty_kernel<<<256, 256, 0, static_cast<hipStream_t>(stream)>>>(static_cast<uint32_t*>(sink));
  return ofq_check_launch();
}

extern "C" int ofq_bench_copy(void* stream, void* dst, const void* src, size_t bytes) {
  if (dst == nullptr || src == nullptr) return OFQ_ERR_NULL_POINTER;
  if (((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15) != 0) {
    return OFQ_ERR_MISALIGNED;
  }
  if (bytes < 16 || bytes % 16 != 0) return OFQ_ERR_BAD_SHAPE;
  const size_t nvec = bytes / 16;
  const size_t blocks = (nvec + 255) / 256;
  if (blocks > 0x7FFFFFFFull) return OFQ_ERR_BAD_SHAPE;
  ofq::copy_kernel<<<(unsigned)blocks, 256, 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<ofq::u32x4*>(dst), static_cast<const ofq::u32x4*>(src), nvec);
  return ofq_check_launch();
}
