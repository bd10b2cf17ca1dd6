// A kernel that only reads: one 16-byte request per lane, the whole buffer in one round, nothing
// computed beyond a value that keeps the loads alive.  What it takes is the time below which no
// kernel that has to read those bytes once can finish; the benchmark reports it beside the GEMVs.
#include "ofq_device.h"
#include "ofq_internal.h"

namespace ofq {
namespace {

__global__ void __launch_bounds__(256)
probe_read_kernel(const u32x4* __restrict__ p, size_t nvec, uint32_t* sink) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const u32x4 v = __builtin_nontemporal_load(p + (i < nvec ? i : nvec - 1));
  const uint32_t a = v[0] ^ v[1] ^ v[2] ^ v[3];
  if (a == 0x9E3779B9u && sink != nullptr) sink[0] = a;  // practically never: keeps the load
}

}  // namespace
}  // namespace ofq

extern "C" int ofq_probe_read(void* stream, const void* buf, size_t bytes, void* sink) {
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
