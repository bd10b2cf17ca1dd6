// min_max_observer, quantization, fake_quantization for gfx950.
//
// Arithmetic follows the reference kernels exactly so that codes are bit-identical:
//   observer      oneflow/user/kernels/min_max_observer_kernel.cpp:22-58 (.cu:117-163)
//   quantization  oneflow/user/kernels/quantization_kernel.cpp:22-62 (.cu:24-95)
//   fake quant    oneflow/user/kernels/fake_quantization_kernel.cpp:22-64 (.cu:24-96)
// i.e. one correctly rounded division, rint (round-half-even), ternary clamps that keep -0.0 and
// NaN as the CPU code does.  hipcc's default fp32 division is the IEEE sequence.
//
// Observer structure: a channel (or the whole tensor) is cut into `splits` slices so that the
// grid has enough blocks to pull full HBM bandwidth; every block reduces its slice's max and
// min with 128-bit loads and wave shuffles and stores one (max,min) pair in the workspace; a
// second tiny launch folds the pairs and does the scale / zero-point arithmetic.  No atomics,
// no initialisation pass, and the result does not depend on block scheduling.
#include <type_traits>
#include "ofq_device.h"

namespace ofq {
namespace {

constexpr int kObsBlock = 256;
constexpr int64_t kObsSliceElems = 4096;  // elements one block reduces: 4 x 16 bytes per thread (fp32)

__host__ __device__ inline int64_t obs_splits(int64_t inner) {
  int64_t s = (inner + kObsSliceElems - 1) / kObsSliceElems;
  return s < 1 ? 1 : s;
}

template<typename T>
__device__ __forceinline__ T t_rint(T v);
template<>
__device__ __forceinline__ float t_rint<float>(float v) {
  return __builtin_rintf(v);
}
template<>
__device__ __forceinline__ double t_rint<double>(double v) {
  return __builtin_rint(v);
}
template<typename T>
__device__ __forceinline__ T t_abs(T v) {
  return v < 0 ? -v : (v == 0 ? (T)0 : v);
}

// scale / zero point of one channel from its extremes
// (oneflow/user/kernels/min_max_observer_kernel.cpp:22-58)
template<typename T>
__device__ __forceinline__ void observer_channel(T vmax, T vmin, int bits, int scheme, int formula,
                                                 T* __restrict__ scale,
                                                 T* __restrict__ zero_point) {
  if (formula == OFQ_FORMULA_CAMBRICON) {
    const T a = t_abs(vmax), b = t_abs(vmin);
    const T m = a < b ? b : a;
    // floor(log2(m)) with log2 evaluated in double and rounded to T, which is what a correctly
    // rounded libm log2 of the CPU kernel returns (min_max_observer_kernel.cpp:55)
    const T lg = (T)log2((double)m);
    *scale = floor(lg) - (T)(bits - 2);
    *zero_point = 0;
  } else if (scheme == OFQ_SCHEME_SYMMETRIC) {
    const T a = t_abs(vmax), b = t_abs(vmin);
    const T m = a < b ? b : a;
    const T denominator = (T)(1 << (bits - 1)) - 1;
    *scale = m / denominator;
    *zero_point = 0;
  } else {
    const T denominator = (T)(1 << bits) - 1;
    const T s = (vmax - vmin) / denominator;
    *scale = s;
    *zero_point = -t_rint<T>(vmin / s);
  }
}

// DIRECT: a channel is a single slice (splits == 1), so the block that reduced it writes its
// scale and zero point itself and no second launch is needed.
template<typename T, bool DIRECT>
__global__ void __launch_bounds__(kObsBlock)
observer_partial(const T* __restrict__ in, int64_t inner, int64_t splits, int64_t total_slices,
                 T* __restrict__ part, int bits, int scheme, int formula, T* __restrict__ scale,
                 T* __restrict__ zero_point) {
  __shared__ T smem[kObsBlock / kWave];
  // slice `blk` of channels * splits; the grid is capped, so a block may take several
  for (int64_t blk = blockIdx.x; blk < total_slices; blk += gridDim.x) {
  const int64_t c = blk / splits;
  const int64_t sp = blk % splits;
  const int64_t begin = sp * kObsSliceElems;
  int64_t end = begin + kObsSliceElems;
  if (end > inner) end = inner;
  const T* p = in + c * inner;
  T vmax = p[begin];
  T vmin = vmax;
  constexpr int V = 16 / sizeof(T);
  // vector body when the slice start is 16-byte aligned
  int64_t i = begin;
  if (((reinterpret_cast<uintptr_t>(p + begin)) & 15u) == 0) {
    const int64_t nvec = (end - begin) / V;
    typedef T vec_t __attribute__((ext_vector_type(V)));
    const vec_t* pv = reinterpret_cast<const vec_t*>(p + begin);
    // all of a thread's loads are requested before the first is used (many blocks with a few
    // 128-bit loads per thread stream better than few blocks with long loops)
    constexpr int kMaxLoads = (int)(kObsSliceElems / V / kObsBlock);
    vec_t x[kMaxLoads];
    bool have[kMaxLoads];
#pragma unroll
    for (int i = 0; i < kMaxLoads; ++i) {
      const int64_t v = threadIdx.x + (int64_t)i * kObsBlock;
      have[i] = v < nvec;
      if (have[i]) x[i] = __builtin_nontemporal_load(pv + v);
    }
#pragma unroll
    for (int i = 0; i < kMaxLoads; ++i) {
      if (!have[i]) continue;
#pragma unroll
      for (int e = 0; e < V; ++e) {
        vmax = OpMax()(vmax, x[i][e]);
        vmin = OpMin()(vmin, x[i][e]);
      }
    }
    i = begin + nvec * V;
  }
  for (int64_t j = i + threadIdx.x; j < end; j += kObsBlock) {
    vmax = OpMax()(vmax, p[j]);
    vmin = OpMin()(vmin, p[j]);
  }
  vmax = block_reduce(vmax, OpMax(), smem);
  vmin = block_reduce(vmin, OpMin(), smem);
  if (threadIdx.x == 0) {
    if (DIRECT) {
      observer_channel<T>(vmax, vmin, bits, scheme, formula, scale + blk, zero_point + blk);
    } else {
      part[2 * blk] = vmax;
      part[2 * blk + 1] = vmin;
    }
  }
  }
}

template<typename T>
__global__ void __launch_bounds__(kObsBlock)
observer_finalize(const T* __restrict__ part, int64_t channels, int64_t splits, int bits,
                  int scheme, int formula, T* __restrict__ scale, T* __restrict__ zero_point) {
  const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  T vmax = part[2 * c * splits];
  T vmin = part[2 * c * splits + 1];
  for (int64_t s = 1; s < splits; ++s) {
    vmax = OpMax()(vmax, part[2 * (c * splits + s)]);
    vmin = OpMin()(vmin, part[2 * (c * splits + s) + 1]);
  }
  observer_channel<T>(vmax, vmin, bits, scheme, formula, scale + c, zero_point + c);
}

// Channels of many slices (a per-layer observer is ONE channel of elem_cnt / 4096 slices): a block
// per channel, the slices strided over its threads.  max / min do not depend on the order.
template<typename T>
__global__ void __launch_bounds__(kObsBlock)
observer_finalize_wide(const T* __restrict__ part, int64_t splits, int bits, int scheme,
                       int formula, T* __restrict__ scale, T* __restrict__ zero_point) {
  __shared__ T smem[kObsBlock / kWave];
  const int64_t c = blockIdx.x;
  const T* p = part + 2 * c * splits;
  T vmax = p[0];
  T vmin = p[1];
  for (int64_t s = threadIdx.x; s < splits; s += kObsBlock) {
    vmax = OpMax()(vmax, p[2 * s]);
    vmin = OpMin()(vmin, p[2 * s + 1]);
  }
  vmax = block_reduce(vmax, OpMax(), smem);
  vmin = block_reduce(vmin, OpMin(), smem);
  if (threadIdx.x == 0) {
    observer_channel<T>(vmax, vmin, bits, scheme, formula, scale + c, zero_point + c);
  }
}

// Very short channels (inner < kObsTinyInner elements, down to one): a thread per channel, so
// that millions of channels do not become millions of blocks.
constexpr int64_t kObsTinyInner = 64;
template<typename T>
__global__ void __launch_bounds__(kObsBlock)
observer_tiny_channels(const T* __restrict__ in, int64_t channels, int64_t inner, int bits,
                       int scheme, int formula, T* __restrict__ scale,
                       T* __restrict__ zero_point) {
  const int64_t step = (int64_t)gridDim.x * kObsBlock;
  for (int64_t c = (int64_t)blockIdx.x * kObsBlock + threadIdx.x; c < channels; c += step) {
    const T* p = in + c * inner;
    T vmax = p[0];
    T vmin = vmax;
    for (int64_t i = 1; i < inner; ++i) {
      vmax = OpMax()(vmax, p[i]);
      vmin = OpMin()(vmin, p[i]);
    }
    observer_channel<T>(vmax, vmin, bits, scheme, formula, scale + c, zero_point + c);
  }
}

// ---- moving_average_min_max_observer ------------------------------------------------------------
// oneflow/user/kernels/moving_average_min_max_observer_kernel.cpp:22-107: while
// current_train_step <= stop_update_after_iters (and training), moving_max / moving_min follow the
// tensor's extremes (first value, then `moving * momentum + extreme * (1 - momentum)`, each
// product and the sum rounded separately); scale / zero_point always come from the moving values.
// The affine zero point rounds half away from zero (std::round, :78), unlike min_max_observer.
// The step counter is read on the device, so the op can be captured in a graph (the reference's
// CUDA kernel copies it to the host first, moving_average_min_max_observer_kernel.cu:249-251).
template<typename T>
__global__ void __launch_bounds__(kWave)
moving_average_finalize(const T* __restrict__ part, int64_t splits,
                        const int64_t* __restrict__ current_train_step,
                        int64_t stop_update_after_iters, int training, float momentum, int bits,
                        int scheme, int formula, T* __restrict__ moving_max,
                        T* __restrict__ moving_min, T* __restrict__ scale,
                        T* __restrict__ zero_point) {
  const bool update = training != 0 && *current_train_step <= stop_update_after_iters;
  T mmax = *moving_max, mmin = *moving_min;
  if (update) {  // uniform
    T vmax = part[0], vmin = part[1];
    for (int64_t s = threadIdx.x; s < splits; s += kWave) {
      vmax = OpMax()(vmax, part[2 * s]);
      vmin = OpMin()(vmin, part[2 * s + 1]);
    }
    vmax = wave_reduce(vmax, OpMax());
    vmin = wave_reduce(vmin, OpMin());
    const T keep = (T)momentum;              // T * float: the float is widened to T
    const T take = (T)(1 - momentum);        // (1 - momentum) is evaluated in float first
    if (formula == OFQ_FORMULA_CAMBRICON || scheme == OFQ_SCHEME_SYMMETRIC) {
      const T a = t_abs(vmax), b = t_abs(vmin);
      const T amax = a < b ? b : a;
      if (mmax == 0) {
        mmax = amax;
      } else {
        const T p0 = mmax * keep, p1 = amax * take;
        mmax = p0 + p1;
      }
      mmin = mmax;  // the symmetric schemes only use moving_max
    } else {
      if (mmax == 0) {
        mmax = vmax;
      } else {
        const T p0 = mmax * keep, p1 = vmax * take;
        mmax = p0 + p1;
      }
      if (mmin == 0) {
        mmin = vmin;
      } else {
        const T p0 = mmin * keep, p1 = vmin * take;
        mmin = p0 + p1;
      }
    }
  }
  if (threadIdx.x != 0) return;
  if (update) {
    *moving_max = mmax;
    *moving_min = mmin;
  }
  if (formula == OFQ_FORMULA_CAMBRICON) {
    const T lg = (T)log2((double)mmax);
    *scale = floor(lg) - (T)(bits - 2);
    *zero_point = 0;
  } else if (scheme == OFQ_SCHEME_SYMMETRIC) {
    const T denominator = (T)(1 << (bits - 1)) - 1;
    *scale = mmax / denominator;
    *zero_point = 0;
  } else {
    const T denominator = (T)(1 << bits) - 1;
    const T sc = (mmax - mmin) / denominator;
    const T r = mmin / sc;
    *scale = sc;
    *zero_point = -(r < 0 ? -floor(-r + (T)0.5) : floor(r + (T)0.5));  // -std::round(r)
  }
}

// ---- quantization / fake quantization ---------------------------------------------------
// IN: element type of `in`; C: type the arithmetic runs in (float for f16/bf16/f32 inputs,
// double for f64); OUT: storage of the result (same as IN, or int8/uint8 codes).
enum { kModeSym = 0, kModeAffineFloatZp = 1, kModeAffineU8Zp = 2 };

template<typename C>
struct QParams {
  C upper, lower;
};

template<typename C, int MODE, bool FAKE, bool RECIP = false>
__device__ __forceinline__ C quant_one(C x, C scale, C zp, C upper, C lower, C recip = 0) {
  C o;
  C q;
  if constexpr (RECIP) {
    q = div_of_half_value(x, scale, recip);
  } else {
    q = x / scale;
  }
  if (MODE == kModeSym) {
    o = t_rint<C>(q);
  } else {
    o = t_rint<C>(q + zp);
  }
  o = o > upper ? upper : o;
  o = o < lower ? lower : o;
  if (FAKE) {
    if (MODE == kModeSym) {
      o = o * scale;
    } else {
      o = (o - zp) * scale;
    }
  }
  return o;
}

template<typename S>
struct Elem;  // load/store helpers keyed by storage type
template<>
struct Elem<float> {
  static __device__ __forceinline__ float ld(const float* p) { return *p; }
  static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
};
template<>
struct Elem<double> {
  static __device__ __forceinline__ double ld(const double* p) { return *p; }
  static __device__ __forceinline__ void st(double* p, double v) { *p = v; }
};
template<>
struct Elem<f16> {
  static __device__ __forceinline__ float ld(const f16* p) { return (float)*p; }
  // The empty asm keeps the narrowing apart from a multiplication that produced v: fused, the
  // compiler emits v_fma_mixlo_f16 with a +0 addend, which turns a product of -0 into +0.
  static __device__ __forceinline__ void st(f16* p, float v) {
    asm volatile("" : "+v"(v));
    *p = (f16)v;
  }
};
template<>
struct Elem<bf16> {
  static __device__ __forceinline__ float ld(const bf16* p) { return bf16_to_float(p->bits); }
  static __device__ __forceinline__ void st(bf16* p, float v) { p->bits = float_to_bf16(v); }
};
template<>
struct Elem<int8_t> {
  // codes are integral and inside [-128,127] after the clamp; NaN (0/0) narrows to 0
  static __device__ __forceinline__ void st(int8_t* p, float v) {
    *p = (v != v) ? (int8_t)0 : (int8_t)(int)v;
  }
};
template<>
struct Elem<uint8_t> {
  static __device__ __forceinline__ void st(uint8_t* p, float v) {
    *p = (v != v) ? (uint8_t)0 : (uint8_t)(int)v;
  }
};

// The zero point as the arithmetic sees it
template<typename C, int MODE>
__device__ __forceinline__ C effective_zp(C zp) {
  if (MODE == kModeAffineU8Zp) {
    // static_cast<uint8_t>(std::round(zp)): round half away from zero, then narrow
    const C r = zp < 0 ? -floor(-zp + (C)0.5) : floor(zp + (C)0.5);
    return (C)(uint8_t)(int)r;
  }
  return zp;
}

// Each lane owns V consecutive elements: 16 bytes of input per load, two loads when the output
// is one byte wide so that the store is 16 bytes too.  The channel of a pack costs a division
// (V | panel, so the whole pack lies in one channel); it is skipped for a per-tensor scale and
// done in 32 bits when the tensor allows it.
template<typename IN, typename C, typename OUT, int MODE, bool FAKE, int V>
__global__ void __launch_bounds__(256)
quantize_kernel(const IN* __restrict__ in, const C* __restrict__ scale,
                const C* __restrict__ zero_point, OUT* __restrict__ out, int64_t elem_cnt,
                int64_t panel, int64_t scale_size, C upper, C lower, int cambricon) {
  const int64_t n_packs = elem_cnt / V;
  const int64_t step = (int64_t)gridDim.x * blockDim.x;
  const bool per_tensor = scale_size == 1;
  const bool small = elem_cnt < 0x7FFFFFFF;
  C s0 = scale[0];
  if (cambricon) s0 = (C)exp2((double)(int)s0);  // scale = 2^int(shift)
  const C zp0 = MODE == kModeSym ? (C)0 : effective_zp<C, MODE>(zero_point[0]);
  // fp16 input and one scale for the tensor: the division becomes a corrected multiplication
  constexpr bool kHalfIn = std::is_same<IN, f16>::value && std::is_same<C, float>::value;
  bool recip_ok = false;
  C recip = 0;
  if constexpr (kHalfIn) {
    const float mag = __builtin_fabsf(s0);
    recip_ok = per_tensor && mag >= 0x1p-60f && mag <= 0x1p60f;  // same for every lane
    if (recip_ok) recip = 1.0f / s0;
  }
  for (int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; p < n_packs; p += step) {
    const int64_t base = p * V;
    C s = s0, zp = zp0;
    if (!per_tensor) {
      int64_t ch = small ? (int64_t)((uint32_t)base / (uint32_t)panel) : base / panel;
      if (ch > scale_size - 1) ch = scale_size - 1;
      s = scale[ch];
      if (cambricon) s = (C)exp2((double)(int)s);
      zp = MODE == kModeSym ? (C)0 : effective_zp<C, MODE>(zero_point[ch]);
    }
    IN xin[V];
    constexpr int kInBytes = V * (int)sizeof(IN);
    if (kInBytes % 16 == 0) {
#pragma unroll
      for (int i = 0; i < kInBytes / 16; ++i) {
        reinterpret_cast<u32x4*>(xin)[i] = __builtin_nontemporal_load(
            reinterpret_cast<const u32x4*>(in + base) + i);
      }
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e) xin[e] = in[base + e];
    }
    OUT r[V];
    if (recip_ok) {
      if constexpr (kHalfIn && sizeof(OUT) == 1 && !FAKE && V % 4 == 0) {
        // byte codes: the clamp moves behind the conversion (v_cvt_i32_f32 saturates and turns
        // NaN into 0, which lies inside every code range), one integer median instead of two
        // compares and two selects, and the bytes are merged in registers
        const int lo = (int)lower, hi = (int)upper;
#pragma unroll
        for (int e4 = 0; e4 < V; e4 += 4) {
          uint32_t b[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float x = (float)Elem<IN>::ld(&xin[e4 + j]);
            float q = div_of_half_value(x, s, recip);
            if (MODE != kModeSym) q = q + zp;
            const float t = t_rint<float>(q);
            int v;
            asm("v_cvt_i32_f32 %0, %1" : "=v"(v) : "v"(t));
            b[j] = (uint32_t)clamp_i32(v, lo, hi);
          }
          // low bytes of b[0..3] -> one word
          const uint32_t lo2 = __builtin_amdgcn_perm(b[1], b[0], 0x0c0c0400u);
          const uint32_t hi2 = __builtin_amdgcn_perm(b[3], b[2], 0x04000c0cu);
          reinterpret_cast<uint32_t*>(r)[e4 / 4] = lo2 | hi2;
        }
      } else if constexpr (kHalfIn) {
#pragma unroll
        for (int e = 0; e < V; ++e) {
          const C x = (C)Elem<IN>::ld(&xin[e]);
          Elem<OUT>::st(&r[e], quant_one<C, MODE, FAKE, true>(x, s, zp, upper, lower, recip));
        }
      }
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e) {
        const C x = (C)Elem<IN>::ld(&xin[e]);
        Elem<OUT>::st(&r[e], quant_one<C, MODE, FAKE>(x, s, zp, upper, lower));
      }
    }
    constexpr int kOutBytes = V * (int)sizeof(OUT);
    if (kOutBytes % 16 == 0) {
#pragma unroll
      for (int i = 0; i < kOutBytes / 16; ++i) {
        __builtin_nontemporal_store(reinterpret_cast<const u32x4*>(r)[i],
                                    reinterpret_cast<u32x4*>(out + base) + i);
      }
    } else if (kOutBytes == 8) {
      *reinterpret_cast<u32x2*>(out + base) = *reinterpret_cast<const u32x2*>(r);
    } else if (kOutBytes == 4) {
      *reinterpret_cast<uint32_t*>(out + base) = *reinterpret_cast<const uint32_t*>(r);
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e) out[base + e] = r[e];
    }
  }
}

// fp16 -> byte codes with one scale for the tensor (the activation quantisation in front of an
// int8 matmul): a wave owns 1024 consecutive elements per turn and takes them as two contiguous
// 1 KB requests (lane l: elements 8l.. and 512 + 8l..), so that every request and both 8-byte
// stores of a wave are whole cache lines; the generic kernel's 32 bytes per lane make each request
// touch half of every line.  elem_cnt a multiple of 1024.  Arithmetic as in quantize_kernel.
// (waves_per_eu: without the cap the scheduler interleaves all 16 quotients of a turn on 96
// registers, 5 waves per SIMD fit instead of 8, and the one-turn-per-wave launch runs in two rounds)
template<typename OUT, int MODE>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(8, 8)))
quantize_half_to_bytes_kernel(const f16* __restrict__ in, const float* __restrict__ scale,
                              const float* __restrict__ zero_point, OUT* __restrict__ out,
                              int64_t tiles, float upper, float lower, int cambricon) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t nwaves = (int64_t)gridDim.x * 4;
  float s = scale[0];
  if (cambricon) s = (float)exp2((double)(int)s);
  const float zp = MODE == kModeSym ? 0.f : effective_zp<float, MODE>(zero_point[0]);
  const float mag = __builtin_fabsf(s);
  const bool recip_ok = mag >= 0x1p-60f && mag <= 0x1p60f;
  const float recip = recip_ok ? 1.0f / s : 0.f;
  const int lo = (int)lower, hi = (int)upper;
  // (the branch on the scale's range is taken once per wave: inside the loop both quotients
  // were computed for every element and one of them selected)
  auto walk = [&](auto fast) {
    for (int64_t tile = wave; tile < tiles; tile += nwaves) {
      const f16* src = in + tile * 1024 + lane * 8;
      u32x4 raw[2];
      raw[0] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src));
      raw[1] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src + 512));
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        const f16x8 xv = __builtin_bit_cast(f16x8, raw[hf]);
        uint32_t words[2];
#pragma unroll
        for (int e4 = 0; e4 < 8; e4 += 4) {
          uint32_t b[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float x = (float)xv[e4 + j];
            float q;
            if constexpr (decltype(fast)::value) {
              q = div_of_half_value(x, s, recip);
            } else {
              q = x / s;
            }
            if (MODE != kModeSym) q = q + zp;
            const float t = t_rint<float>(q);
            int v;
            asm("v_cvt_i32_f32 %0, %1" : "=v"(v) : "v"(t));  // saturates; NaN -> 0
            b[j] = (uint32_t)clamp_i32(v, lo, hi);
          }
          const uint32_t lo2 = __builtin_amdgcn_perm(b[1], b[0], 0x0c0c0400u);
          const uint32_t hi2 = __builtin_amdgcn_perm(b[3], b[2], 0x04000c0cu);
          words[e4 / 4] = lo2 | hi2;
        }
        u32x2 w2 = {words[0], words[1]};
        __builtin_nontemporal_store(
            w2, reinterpret_cast<u32x2*>(out + tile * 1024 + hf * 512 + lane * 8));
      }
    }
  };
  if (recip_ok) {
    walk(std::true_type());
  } else {
    walk(std::false_type());
  }
}

inline int grid_for(int64_t items, int block) {
  int64_t g = (items + block - 1) / block;
  const int64_t cap = 256 * 32;
  if (g > cap) g = cap;
  if (g < 1) g = 1;
  return (int)g;
}

template<typename IN, typename C, typename OUT, int MODE, bool FAKE>
int launch_quant(hipStream_t st, const void* in, const void* scale, const void* zp, void* out,
                 int64_t elem_cnt, int64_t panel, int64_t scale_size, C upper, C lower,
                 int cambricon) {
  // 16 bytes of input per lane (4 floats, 2 doubles, 8 halves); 32 when the output is bytes and
  // the input halves, so that loads and the store are all 128-bit
  constexpr int V = (sizeof(OUT) == 1 && sizeof(IN) == 2) ? 16 : 16 / (int)sizeof(IN);
  const IN* i = static_cast<const IN*>(in);
  OUT* o = static_cast<OUT*>(out);
  const C* s = static_cast<const C*>(scale);
  const C* z = static_cast<const C*>(zp);
  if constexpr (std::is_same<IN, f16>::value && std::is_same<C, float>::value && sizeof(OUT) == 1
                && !FAKE) {
    if (scale_size == 1 && elem_cnt % 1024 == 0) {
      const int64_t tiles = elem_cnt / 1024;
      quantize_half_to_bytes_kernel<OUT, MODE><<<grid_for(tiles, 4), 256, 0, st>>>(
          i, s, z, o, tiles, upper, lower, cambricon);
      return ofq_check_launch();
    }
  }
  if (panel % V == 0 && elem_cnt % V == 0) {
    quantize_kernel<IN, C, OUT, MODE, FAKE, V><<<grid_for(elem_cnt / V, 256), 256, 0, st>>>(
        i, s, z, o, elem_cnt, panel, scale_size, upper, lower, cambricon);
  } else {
    quantize_kernel<IN, C, OUT, MODE, FAKE, 1><<<grid_for(elem_cnt, 256), 256, 0, st>>>(
        i, s, z, o, elem_cnt, panel, scale_size, upper, lower, cambricon);
  }
  return ofq_check_launch();
}

template<typename IN, typename C, typename OUT, bool FAKE>
int dispatch_mode(hipStream_t st, const void* in, const void* scale, const void* zp, void* out,
                  int64_t elem_cnt, int64_t panel, int64_t scale_size, int bits, int scheme,
                  int formula, int zp_mode) {
  const bool cambricon = formula == OFQ_FORMULA_CAMBRICON;
  if (cambricon || scheme == OFQ_SCHEME_SYMMETRIC) {
    const C upper = (C)(1 << (bits - 1)) - 1;
    const C lower = -upper - 1;
    return launch_quant<IN, C, OUT, kModeSym, FAKE>(st, in, scale, zp, out, elem_cnt, panel,
                                                    scale_size, upper, lower, cambricon);
  }
  const C upper = (C)(1 << bits) - 1;
  const C lower = 0;
  if (zp_mode == OFQ_ZP_UINT8) {
    return launch_quant<IN, C, OUT, kModeAffineU8Zp, FAKE>(st, in, scale, zp, out, elem_cnt,
                                                           panel, scale_size, upper, lower, 0);
  }
  return launch_quant<IN, C, OUT, kModeAffineFloatZp, FAKE>(st, in, scale, zp, out, elem_cnt,
                                                            panel, scale_size, upper, lower, 0);
}

int check_quant_args(const void* in, const void* scale, const void* zero_point, const void* out,
                     int64_t elem_cnt, int64_t scale_size, int bits, int scheme, int formula,
                     int zp_mode) {
  // attribute domain: oneflow/user/ops/quantization_op.cpp:92-104
  OFQ_RETURN_IF(bits <= 1 || bits > 8, OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(scheme != OFQ_SCHEME_SYMMETRIC && scheme != OFQ_SCHEME_AFFINE, OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(formula != OFQ_FORMULA_GOOGLE && formula != OFQ_FORMULA_CAMBRICON,
                OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(zp_mode != OFQ_ZP_FLOAT && zp_mode != OFQ_ZP_UINT8, OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(elem_cnt < 0 || scale_size < 1, OFQ_ERR_BAD_SHAPE);
  OFQ_RETURN_IF(scale_size > 1 && (elem_cnt % scale_size) != 0, OFQ_ERR_BAD_SHAPE);
  if (elem_cnt == 0) return OFQ_OK;
  OFQ_RETURN_IF(in == nullptr || scale == nullptr || out == nullptr, OFQ_ERR_NULL_POINTER);
  OFQ_RETURN_IF(formula == OFQ_FORMULA_GOOGLE && scheme == OFQ_SCHEME_AFFINE
                    && zero_point == nullptr,
                OFQ_ERR_NULL_POINTER);
  OFQ_RETURN_IF(!ofq_aligned16(in) || !ofq_aligned16(out), OFQ_ERR_MISALIGNED);
  return OFQ_OK;
}

}  // namespace
template<typename T>
int launch_observer(hipStream_t st, const void* in, void* workspace, void* scale,
                    void* zero_point, int64_t channels, int64_t inner, int64_t splits, int bits,
                    int scheme, int formula) {
  const T* src = static_cast<const T*>(in);
  T* sc = static_cast<T*>(scale);
  T* zp = static_cast<T*>(zero_point);
  constexpr int64_t kMaxGrid = 1 << 22;  // blocks; beyond, a block walks several slices
  if (inner < kObsTinyInner) {
    int64_t grid = (channels + kObsBlock - 1) / kObsBlock;
    if (grid > kMaxGrid) grid = kMaxGrid;
    observer_tiny_channels<T><<<(int)grid, kObsBlock, 0, st>>>(src, channels, inner, bits, scheme,
                                                              formula, sc, zp);
    return ofq_check_launch();
  }
  const int64_t total = channels * splits;
  const int grid = (int)(total < kMaxGrid ? total : kMaxGrid);
  if (splits == 1) {
    observer_partial<T, true><<<grid, kObsBlock, 0, st>>>(src, inner, 1, total, nullptr, bits,
                                                         scheme, formula, sc, zp);
    return ofq_check_launch();
  }
  T* part = static_cast<T*>(workspace);
  observer_partial<T, false><<<grid, kObsBlock, 0, st>>>(src, inner, splits, total, part, bits,
                                                        scheme, formula, nullptr, nullptr);
  if (splits > 32 && channels <= kMaxGrid) {
    observer_finalize_wide<T><<<(int)channels, kObsBlock, 0, st>>>(part, splits, bits, scheme,
                                                                  formula, sc, zp);
  } else {
    const int fin_grid = (int)((channels + kObsBlock - 1) / kObsBlock);
    observer_finalize<T><<<fin_grid, kObsBlock, 0, st>>>(part, channels, splits, bits, scheme,
                                                         formula, sc, zp);
  }
  return ofq_check_launch();
}

}  // namespace ofq

using namespace ofq;

extern "C" size_t ofq_min_max_observer_workspace_bytes(int in_dtype, int64_t elem_cnt,
                                                       int64_t channels) {
  if (channels <= 0 || elem_cnt <= 0) return 0;
  const size_t es = in_dtype == OFQ_F64 ? 8 : 4;
  const int64_t inner = elem_cnt / channels;
  return (size_t)(channels * obs_splits(inner)) * 2 * es;
}

extern "C" int ofq_min_max_observer(void* stream, const void* in, void* scale, void* zero_point,
                                    int in_dtype, int64_t elem_cnt, int64_t channels,
                                    int quantization_bit, int scheme, int formula,
                                    void* workspace, size_t workspace_bytes) {
  // attribute domain: oneflow/user/ops/min_max_observer_op.cpp:58-70
  OFQ_RETURN_IF(quantization_bit <= 1 || quantization_bit > 8, OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(scheme != OFQ_SCHEME_SYMMETRIC && scheme != OFQ_SCHEME_AFFINE, OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(formula != OFQ_FORMULA_GOOGLE && formula != OFQ_FORMULA_CAMBRICON,
                OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(in_dtype != OFQ_F32 && in_dtype != OFQ_F64, OFQ_ERR_BAD_DTYPE);
  OFQ_RETURN_IF(channels < 1 || elem_cnt < 1 || elem_cnt % channels != 0, OFQ_ERR_BAD_SHAPE);
  // per-channel mode is not supported in cambricon scheme: min_max_observer_kernel.cpp:105-108
  OFQ_RETURN_IF(formula == OFQ_FORMULA_CAMBRICON && channels != 1, OFQ_ERR_UNSUPPORTED);
  OFQ_RETURN_IF(in == nullptr || scale == nullptr || zero_point == nullptr, OFQ_ERR_NULL_POINTER);
  OFQ_RETURN_IF(!ofq_aligned16(in), OFQ_ERR_MISALIGNED);
  const size_t need = ofq_min_max_observer_workspace_bytes(in_dtype, elem_cnt, channels);
  OFQ_RETURN_IF(workspace == nullptr || workspace_bytes < need, OFQ_ERR_WORKSPACE);
  const int64_t inner = elem_cnt / channels;
  const int64_t splits = obs_splits(inner);
  OFQ_RETURN_IF(channels * splits > 0x7FFFFFFF, OFQ_ERR_BAD_SHAPE);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (in_dtype == OFQ_F32) {
    return launch_observer<float>(st, in, workspace, scale, zero_point, channels, inner, splits,
                                  quantization_bit, scheme, formula);
  }
  return launch_observer<double>(st, in, workspace, scale, zero_point, channels, inner, splits,
                                 quantization_bit, scheme, formula);
}

extern "C" size_t ofq_moving_average_min_max_observer_workspace_bytes(int in_dtype,
                                                                      int64_t elem_cnt) {
  return ofq_min_max_observer_workspace_bytes(in_dtype, elem_cnt, 1);
}

extern "C" int ofq_moving_average_min_max_observer(
    void* stream, const void* in, const int64_t* current_train_step, void* moving_max,
    void* moving_min, void* scale, void* zero_point, int in_dtype, int64_t elem_cnt,
    int quantization_bit, int scheme, int formula, float momentum,
    int64_t stop_update_after_iters, int training, void* workspace, size_t workspace_bytes) {
  // attribute domain: oneflow/user/ops/moving_average_min_max_observer_op.cpp:72-86
  OFQ_RETURN_IF(quantization_bit <= 1 || quantization_bit > 8, OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(scheme != OFQ_SCHEME_SYMMETRIC && scheme != OFQ_SCHEME_AFFINE, OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(formula != OFQ_FORMULA_GOOGLE && formula != OFQ_FORMULA_CAMBRICON,
                OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(stop_update_after_iters <= 0, OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(in_dtype != OFQ_F32 && in_dtype != OFQ_F64, OFQ_ERR_BAD_DTYPE);
  OFQ_RETURN_IF(elem_cnt < 1, OFQ_ERR_BAD_SHAPE);
  OFQ_RETURN_IF(in == nullptr || current_train_step == nullptr || moving_max == nullptr
                    || moving_min == nullptr || scale == nullptr || zero_point == nullptr,
                OFQ_ERR_NULL_POINTER);
  OFQ_RETURN_IF(!ofq_aligned16(in), OFQ_ERR_MISALIGNED);
  const size_t need = ofq_moving_average_min_max_observer_workspace_bytes(in_dtype, elem_cnt);
  OFQ_RETURN_IF(workspace == nullptr || workspace_bytes < need, OFQ_ERR_WORKSPACE);
  const int64_t splits = obs_splits(elem_cnt);
  OFQ_RETURN_IF(splits > 0x7FFFFFFF, OFQ_ERR_BAD_SHAPE);
  hipStream_t st = static_cast<hipStream_t>(stream);
  // The extremes are reduced whether or not this step updates the moving values: whether it does
  // is known on the device only.
  if (in_dtype == OFQ_F32) {
    observer_partial<float, false><<<(int)splits, kObsBlock, 0, st>>>(
        static_cast<const float*>(in), elem_cnt, splits, splits, static_cast<float*>(workspace), 0,
        0, 0, nullptr, nullptr);
    moving_average_finalize<float><<<1, kWave, 0, st>>>(
        static_cast<const float*>(workspace), splits, current_train_step, stop_update_after_iters,
        training, momentum, quantization_bit, scheme, formula, static_cast<float*>(moving_max),
        static_cast<float*>(moving_min), static_cast<float*>(scale),
        static_cast<float*>(zero_point));
  } else {
    observer_partial<double, false><<<(int)splits, kObsBlock, 0, st>>>(
        static_cast<const double*>(in), elem_cnt, splits, splits, static_cast<double*>(workspace),
        0, 0, 0, nullptr, nullptr);
    moving_average_finalize<double><<<1, kWave, 0, st>>>(
        static_cast<const double*>(workspace), splits, current_train_step,
        stop_update_after_iters, training, momentum, quantization_bit, scheme, formula,
        static_cast<double*>(moving_max), static_cast<double*>(moving_min),
        static_cast<double*>(scale), static_cast<double*>(zero_point));
  }
  return ofq_check_launch();
}

extern "C" int ofq_quantization(void* stream, const void* in, const void* scale,
                                const void* zero_point, void* out, int in_dtype, int out_dtype,
                                int64_t elem_cnt, int64_t scale_size, int quantization_bit,
                                int scheme, int formula, int zp_mode) {
  int rc = check_quant_args(in, scale, zero_point, out, elem_cnt, scale_size, quantization_bit,
                            scheme, formula, zp_mode);
  if (rc != OFQ_OK || elem_cnt == 0) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t panel = scale_size > 1 ? elem_cnt / scale_size : elem_cnt;
  const bool integer_out = out_dtype == OFQ_I8 || out_dtype == OFQ_U8;
  if (integer_out) {
    // signed codes for the symmetric range [-2^(b-1), 2^(b-1)-1], unsigned for [0, 2^b-1]
    const bool sym = scheme == OFQ_SCHEME_SYMMETRIC || formula == OFQ_FORMULA_CAMBRICON;
    OFQ_RETURN_IF(sym != (out_dtype == OFQ_I8), OFQ_ERR_BAD_DTYPE);
  } else {
    OFQ_RETURN_IF(out_dtype != in_dtype, OFQ_ERR_BAD_DTYPE);
  }
#define OFQ_Q(IN, C, OUT)                                                                       \
  return dispatch_mode<IN, C, OUT, false>(st, in, scale, zero_point, out, elem_cnt, panel,      \
                                          scale_size, quantization_bit, scheme, formula, zp_mode)
  switch (in_dtype) {
    case OFQ_F32:
      if (out_dtype == OFQ_I8) OFQ_Q(float, float, int8_t);
      if (out_dtype == OFQ_U8) OFQ_Q(float, float, uint8_t);
      OFQ_Q(float, float, float);
    case OFQ_F64:
      OFQ_RETURN_IF(integer_out, OFQ_ERR_UNSUPPORTED);
      OFQ_Q(double, double, double);
    case OFQ_F16:
      if (out_dtype == OFQ_I8) OFQ_Q(f16, float, int8_t);
      if (out_dtype == OFQ_U8) OFQ_Q(f16, float, uint8_t);
      OFQ_Q(f16, float, f16);
    case OFQ_BF16:
      if (out_dtype == OFQ_I8) OFQ_Q(bf16, float, int8_t);
      if (out_dtype == OFQ_U8) OFQ_Q(bf16, float, uint8_t);
      OFQ_Q(bf16, float, bf16);
    default: return OFQ_ERR_BAD_DTYPE;
  }
#undef OFQ_Q
}

extern "C" int ofq_fake_quantization(void* stream, const void* in, const void* scale,
                                     const void* zero_point, void* out, int in_dtype,
                                     int64_t elem_cnt, int64_t scale_size, int quantization_bit,
                                     int scheme, int formula, int zp_mode) {
  int rc = check_quant_args(in, scale, zero_point, out, elem_cnt, scale_size, quantization_bit,
                            scheme, formula, zp_mode);
  if (rc != OFQ_OK || elem_cnt == 0) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t panel = scale_size > 1 ? elem_cnt / scale_size : elem_cnt;
#define OFQ_FQ(IN, C)                                                                          \
  return dispatch_mode<IN, C, IN, true>(st, in, scale, zero_point, out, elem_cnt, panel,       \
                                        scale_size, quantization_bit, scheme, formula, zp_mode)
  switch (in_dtype) {
    case OFQ_F32: OFQ_FQ(float, float);
    case OFQ_F64: OFQ_FQ(double, double);
    case OFQ_F16: OFQ_FQ(f16, float);
    case OFQ_BF16: OFQ_FQ(bf16, float);
    default: return OFQ_ERR_BAD_DTYPE;
  }
#undef OFQ_FQ
}
