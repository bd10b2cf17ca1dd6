// Shared device-side helpers for the gfx950 kernels: element types, rounding to T, wave and
// block reductions.  HIP only; compiled with -ffp-contract=off so that `a * b + c` written in
// source rounds twice -- fused multiply-adds are always spelled out with a builtin.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ofq.h"

namespace ofq {

typedef _Float16 f16;
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned short u16x8 __attribute__((ext_vector_type(8)));

constexpr int kWave = 64;

// bf16 is carried as its bit pattern; arithmetic is fp32 followed by one rounding.
struct bf16 {
  uint16_t bits;
};

__device__ __forceinline__ float bf16_to_float(uint16_t b) {
  return __builtin_bit_cast(float, (uint32_t)b << 16);
}
// round-to-nearest-even; lowers to v_cvt_pk_bf16_f32 on gfx950
__device__ __forceinline__ uint16_t float_to_bf16(float f) {
  return __builtin_bit_cast(uint16_t, (__bf16)f);
}

// Element-type traits: T <-> float, and "arithmetic in T" (one rounding per operation).
template<typename T>
struct TT;

template<>
struct TT<float> {
  typedef float storage;
  static constexpr int dtype = OFQ_F32;
  static __device__ __forceinline__ float load(const float* p) { return *p; }
  static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
  static __device__ __forceinline__ float round(float v) { return v; }
};
template<>
struct TT<f16> {
  typedef f16 storage;
  static constexpr int dtype = OFQ_F16;
  static __device__ __forceinline__ float load(const f16* p) { return (float)*p; }
  static __device__ __forceinline__ void store(f16* p, float v) { *p = (f16)v; }
  static __device__ __forceinline__ float round(float v) { return (float)(f16)v; }
};
template<>
struct TT<bf16> {
  typedef uint16_t storage;
  static constexpr int dtype = OFQ_BF16;
  static __device__ __forceinline__ float load(const uint16_t* p) { return bf16_to_float(*p); }
  static __device__ __forceinline__ void store(uint16_t* p, float v) { *p = float_to_bf16(v); }
  static __device__ __forceinline__ float round(float v) {
    return bf16_to_float(float_to_bf16(v));
  }
};

// raw bits of a 16-bit T -> float.  Registers that hold scales between their load and their use
// keep them as uint16_t: arrays of f16 inside a struct can end up in scratch memory.
template<typename T>
__device__ __forceinline__ float raw16_to_float(uint16_t raw) {
  if constexpr (TT<T>::dtype == OFQ_BF16) {
    return __builtin_bit_cast(float, (uint32_t)raw << 16);
  } else {
    return (float)__builtin_bit_cast(f16, raw);
  }
}

// ---- wave64 reductions through DPP-free cross-lane shuffles (ds_bpermute / permlane) ----
template<typename V, typename Op>
__device__ __forceinline__ V wave_reduce(V v, Op op) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) { v = op(v, __shfl_xor(v, off, kWave)); }
  return v;
}

struct OpSum {
  template<typename V>
  __device__ __forceinline__ V operator()(V a, V b) const {
    return a + b;
  }
};
struct OpMax {
  __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); }
  __device__ __forceinline__ double operator()(double a, double b) const { return fmax(a, b); }
};
struct OpMin {
  __device__ __forceinline__ float operator()(float a, float b) const { return fminf(a, b); }
  __device__ __forceinline__ double operator()(double a, double b) const { return fmin(a, b); }
};

// Block-wide reduction; `smem` needs blockDim.x/64 elements; every thread gets the result.
template<typename V, typename Op>
__device__ __forceinline__ V block_reduce(V v, Op op, V* smem) {
  v = wave_reduce(v, op);
  const int wave = threadIdx.x / kWave;
  const int nwaves = blockDim.x / kWave;
  __syncthreads();  // smem may still be read from a previous reduction
  if ((threadIdx.x & (kWave - 1)) == 0) smem[wave] = v;
  __syncthreads();
  V r = smem[0];
  for (int i = 1; i < nwaves; ++i) r = op(r, smem[i]);
  return r;
}

// integer code of element `idx` of a packed tensor (flat index over the UNPACKED shape):
// 4-bit: element 2i is the high nibble of byte i; an int8 container sign-extends the nibble.
template<int BITS, bool SIGNED>
__device__ __forceinline__ int code_at(const uint8_t* q, int64_t idx) {
  if (BITS == 8) { return SIGNED ? (int)(int8_t)q[idx] : (int)q[idx]; }
  const uint8_t byte = q[idx >> 1];
  const int nib = (idx & 1) ? (byte & 0xF) : (byte >> 4);
  return SIGNED ? ((nib ^ 8) - 8) : nib;
}

// a / b for a that came from an fp16 value and a reciprocal y = 1 / b formed once per scale (IEEE
// division), b within [2^-60, 2^60]: the product a * y corrected twice with the exact remainder
// (Markstein's division steps) is the correctly rounded quotient, bit for bit what `a / b`
// gives, at 5 fused operations instead of the 11 of the division sequence the compiler emits
// (which made the fp16 -> int8 kernel compute-bound).  Nothing over- or underflows: |a| is 0 or
// in [2^-24, 65504].  Zero keeps its sign through a * y, infinity and NaN their class.
__device__ __forceinline__ float div_of_half_value(float a, float b, float y) {
  const float q0 = a * y;
  const float r0 = __builtin_fmaf(-b, q0, a);
  const float q1 = __builtin_fmaf(r0, y, q0);
  const float r1 = __builtin_fmaf(-b, q1, a);
  const float q = __builtin_fmaf(r1, y, q1);
  // normal or subnormal a (class bits 3, 4, 7, 8): the corrected quotient
  return __builtin_amdgcn_classf(a, 0x198) ? q : q0;
}

// The same quotient for a caller that only rounds it to an integer code and knows a is not
// infinite: the select above is there for a = +-inf alone (the remainders turn it into NaN); NaN
// stays NaN either way, and a zero comes out as +0 instead of +-0, which no integer code tells
// apart.
__device__ __forceinline__ float div_of_finite_half_value(float a, float b, float y) {
  const float q0 = a * y;
  const float r0 = __builtin_fmaf(-b, q0, a);
  const float q1 = __builtin_fmaf(r0, y, q0);
  const float r1 = __builtin_fmaf(-b, q1, a);
  return __builtin_fmaf(r1, y, q1);
}

// min(max(v, lo), hi) for lo <= hi in one instruction (the compiler cannot know lo <= hi and
// emits the pair)
__device__ __forceinline__ int clamp_i32(int v, int lo, int hi) {
  int r;
  asm("v_med3_i32 %0, %1, %2, %3" : "=v"(r) : "v"(v), "v"(lo), "v"(hi));
  return r;
}

}  // namespace ofq

// host-side launch helpers -------------------------------------------------------------------
#define OFQ_RETURN_IF(cond, status) \
  do {                              \
    if (cond) return (status);      \
  } while (0)

// The runtime's record of a failed launch is read (and thereby cleared) here; it is kept for the
// caller's own asynchronous-error query (ofq_hip_get_async_error, hip_shim.hip).
namespace ofq {
void note_launch_error(int hip_error);
}
static inline int ofq_check_launch() {
  const hipError_t e = hipGetLastError();
  if (e == hipSuccess) return OFQ_OK;
  ofq::note_launch_error((int)e);
  return OFQ_ERR_LAUNCH;
}
static inline bool ofq_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// A kernel that uses more than 64 KB of dynamic LDS has to be allowed to once per device.
// `done` holds one bit per device ordinal (a function-local static of the launcher, one per
// kernel instantiation); the call is idempotent, so two threads racing here at worst both make it.
#include <atomic>
static inline bool ofq_allow_dynamic_lds(const void* kernel, int bytes, std::atomic<uint64_t>& done) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return false;
  const uint64_t bit = 1ull << (dev & 63);
  if (done.load(std::memory_order_acquire) & bit) return true;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) {
    return false;
  }
  done.fetch_or(bit, std::memory_order_release);
  return true;
}
