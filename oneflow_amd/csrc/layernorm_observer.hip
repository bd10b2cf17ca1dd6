// fused_layer_norm_min_max_observer for gfx950: LayerNorm over the last axis fused with a
// per-tensor symmetric min/max observer of the normalised output.
//
// LayerNorm arithmetic (oneflow/core/cuda/layer_norm.cuh:212-233,377-380 and the affine store of
// oneflow/user/kernels/layer_norm_gpu_kernel.cu:40-70): statistics in fp32,
// var = max(M2/n, 0), inv = rsqrt(var + eps); the normalised value is rounded to T first and the
// affine `* gamma + beta` is then carried out in T (two more roundings).
// Observer (oneflow/user/kernels/min_max_observer_kernel.cu:117-131): scale = absmax / (2^(b-1)-1).
// With SKIP the normalised input is that of skip_layer_norm
// (oneflow/user/kernels/skip_layer_norm_kernel.cu:36-67): (x + bias[c]) + skip * T(alpha), every
// operation rounded to T, an absent bias or skip entering as zero.
//
// Rows of up to 4096 elements: one WAVE per row.  The row is read from HBM once (128-bit loads,
// 1 KB per wave instruction) and kept in registers for the three uses (sum, squared deviations,
// normalise); the reductions are cross-lane only, so no barrier and no LDS is involved and the
// waves of a CU drift apart, which overlaps one wave's loads with another's stores.  Longer rows
// use one block per row.  The absmax of the stored values goes to the workspace (one float per
// wave or per row) and a second one-wave launch folds them and divides.
#include <atomic>
#include <type_traits>
#include "ofq_device.h"

// Scratch of the entry point that allocates nothing (ofq_fused_layer_norm_min_max_observer_static):
// one partial absmax per row or wave, the role the caller's workspace plays in the other entry
// points.  Every device the library runs on holds its own copy until the process ends.  In host
// code the name below is only a handle for hipGetSymbolAddress; the device address it yields is
// what kernels and copies are given.
#define OFQ_LN_STATIC_MAX_ROWS 65536
static __device__ __align__(256) float scratch[OFQ_LN_STATIC_MAX_ROWS];

namespace ofq {
namespace {

constexpr int kLnBlock = 256;

template<typename T>
struct Pack8 {
  typename TT<T>::storage v[8];
};

template<typename T>
__device__ __forceinline__ void load8(const typename TT<T>::storage* p, float* f) {
  typedef typename TT<T>::storage S;
  S tmp[8];
  if (sizeof(S) == 2) {
    *reinterpret_cast<u32x4*>(tmp) = *reinterpret_cast<const u32x4*>(p);
  } else {
    reinterpret_cast<u32x4*>(tmp)[0] = reinterpret_cast<const u32x4*>(p)[0];
    reinterpret_cast<u32x4*>(tmp)[1] = reinterpret_cast<const u32x4*>(p)[1];
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) f[e] = TT<T>::load(&tmp[e]);
}

template<typename T>
__device__ __forceinline__ void store8(typename TT<T>::storage* p, const float* f) {
  typedef typename TT<T>::storage S;
  S tmp[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) TT<T>::store(&tmp[e], f[e]);
  if (sizeof(S) == 2) {
    *reinterpret_cast<u32x4*>(p) = *reinterpret_cast<const u32x4*>(tmp);
  } else {
    reinterpret_cast<u32x4*>(p)[0] = reinterpret_cast<const u32x4*>(tmp)[0];
    reinterpret_cast<u32x4*>(p)[1] = reinterpret_cast<const u32x4*>(tmp)[1];
  }
}

// the residual inputs of skip_layer_norm; alpha already rounded to T
template<typename T>
struct SkipArgs {
  const typename TT<T>::storage* bias;  // [cols] or null
  const typename TT<T>::storage* skip;  // [rows, cols] or null
  float alpha;
};

// T((x - mean) * inv) as the reference forms it: the fp32 product, rounded to fp32, is narrowed
// to T (layer_norm.cuh stores through static_cast).  The empty asm keeps the two roundings
// apart: fused into v_fma_mixlo_f16 the product would be rounded to fp16 once, which differs in
// about one element of 30000.
template<typename T>
__device__ __forceinline__ float normalised(float d, float inv) {
  float p = d * inv;
  if constexpr (TT<T>::dtype == OFQ_F16) asm volatile("" : "+v"(p));
  return TT<T>::round(p);
}

template<typename T>
__device__ __forceinline__ float skip_sum(float x, float b, float s, float alpha) {
  return TT<T>::round(TT<T>::round(x + b) + TT<T>::round(s * alpha));
}

// EXACT statistics: the row sum and the squared deviations from the unrounded mean are taken in
// fp64 (a sum of fp16 / bf16 values of ordinary range is exact there in any order, the squares
// carry errors of 1e-16), and mean and inv are each rounded once to the fp32 values the
// normalisation uses -- the correctly rounded statistics of the row, independent of the order of
// summation.  The fp32 statistics (the default) depend on that order in the last bit, as the
// reference's own do.  The cost is three fp64 operations per element and pass.
__device__ __forceinline__ float exact_inv(double m2, double n, double eps) {
  double var = m2 / n;
  if (var < 0.0) var = 0.0;
  return (float)(1.0 / __builtin_sqrt(var + eps));
}

// NP = packs of 8 elements each lane caches; cols <= kLnBlock * 8 * NP and 8 | cols.
template<typename T, int NP, bool SKIP, bool EXACT>
__global__ void __launch_bounds__(kLnBlock)
ln_observer_rows(const typename TT<T>::storage* __restrict__ x,
                 const typename TT<T>::storage* __restrict__ gamma,
                 const typename TT<T>::storage* __restrict__ beta,
                 typename TT<T>::storage* __restrict__ y, float* __restrict__ row_absmax,
                 int64_t cols, double eps64, SkipArgs<T> sk) {
  __shared__ float smem[kLnBlock / kWave];
  __shared__ double smem64[EXACT ? kLnBlock / kWave : 1];
  const float eps = (float)eps64;
  const int64_t row = blockIdx.x;
  const typename TT<T>::storage* xr = x + row * cols;
  typename TT<T>::storage* yr = y + row * cols;
  const int npacks = (int)(cols / 8);
  float v[NP][8];
  float sum = 0.0f;
  double sum64 = 0.0;
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const int p = threadIdx.x + i * kLnBlock;
    if (p < npacks) {
      load8<T>(xr + (int64_t)p * 8, v[i]);
      if (SKIP) {
        float bb[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        float ss[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (sk.bias) load8<T>(sk.bias + (int64_t)p * 8, bb);
        if (sk.skip) load8<T>(sk.skip + row * cols + (int64_t)p * 8, ss);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[i][e] = skip_sum<T>(v[i][e], bb[e], ss[e], sk.alpha);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if constexpr (EXACT) sum64 += (double)v[i][e];
        else sum += v[i][e];
      }
    }
  }
  float mean, inv;
  if constexpr (EXACT) {
    sum64 = block_reduce(sum64, OpSum(), smem64);
    const double mean64 = sum64 / (double)cols;
    double q = 0.0;
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      const int p = threadIdx.x + i * kLnBlock;
      if (p < npacks) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const double d = (double)v[i][e] - mean64;
          q = __builtin_fma(d, d, q);
        }
      }
    }
    q = block_reduce(q, OpSum(), smem64);
    mean = (float)mean64;
    inv = exact_inv(q, (double)cols, eps64);
  } else {
    sum = block_reduce(sum, OpSum(), smem);
    mean = sum / (float)cols;
    float m2 = 0.0f;
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      const int p = threadIdx.x + i * kLnBlock;
      if (p < npacks) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float d = v[i][e] - mean;
          m2 = __builtin_fmaf(d, d, m2);
        }
      }
    }
    m2 = block_reduce(m2, OpSum(), smem);
    const float var = fmaxf(m2 / (float)cols, 0.0f);
    inv = 1.0f / __builtin_sqrtf(var + eps);
  }
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const int p = threadIdx.x + i * kLnBlock;
    if (p < npacks) {
      float g[8], b[8], o[8];
      if (gamma) load8<T>(gamma + (int64_t)p * 8, g);
      if (beta) load8<T>(beta + (int64_t)p * 8, b);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float t = normalised<T>(v[i][e] - mean, inv);
        if (gamma) t = TT<T>::round(t * g[e]);
        if (beta) t = TT<T>::round(t + b[e]);
        else if (gamma) t = t + 0.0f;  // the reference adds its default beta 0: -0 becomes +0
        o[e] = t;
        amax = fmaxf(amax, fabsf(t));
      }
      store8<T>(yr + (int64_t)p * 8, o);
    }
  }
  amax = block_reduce(amax, OpMax(), smem);
  if (threadIdx.x == 0) row_absmax[row] = amax;
}

// Raw 8-element packs (16 bytes of fp16/bf16, 32 bytes of fp32) and their widening to fp32.
template<typename T>
struct RawPack {
  u32x4 q[sizeof(typename TT<T>::storage) * 8 / 16];
};
template<typename T>
__device__ __forceinline__ RawPack<T> load_raw(const typename TT<T>::storage* p) {
  RawPack<T> r;
#pragma unroll
  for (int i = 0; i < (int)(sizeof(r.q) / 16); ++i) r.q[i] = reinterpret_cast<const u32x4*>(p)[i];
  return r;
}
// (whole-vector bit casts: element access through the struct member, `r.q[0][w]`, came out of the
// compiler as component 0 for every w)
template<typename T>
__device__ __forceinline__ void widen(const RawPack<T>& r, float* f) {
  if constexpr (TT<T>::dtype == OFQ_F16) {
    const f16x8 h = __builtin_bit_cast(f16x8, r.q[0]);
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = (float)h[i];
  } else if constexpr (TT<T>::dtype == OFQ_BF16) {
    const u16x8 h = __builtin_bit_cast(u16x8, r.q[0]);
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = bf16_to_float(h[i]);
  } else {
    const f32x4 lo = __builtin_bit_cast(f32x4, r.q[0]);
    const f32x4 hi = __builtin_bit_cast(f32x4, r.q[sizeof(r.q) / 16 - 1]);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[i] = lo[i];
      f[4 + i] = hi[i];
    }
  }
}

template<typename T>
__device__ __forceinline__ RawPack<T> narrow(const float* f) {
  RawPack<T> r;
  if constexpr (TT<T>::dtype == OFQ_F16) {
    f16x8 h;
#pragma unroll
    for (int i = 0; i < 8; ++i) h[i] = (f16)f[i];
    r.q[0] = __builtin_bit_cast(u32x4, h);
  } else if constexpr (TT<T>::dtype == OFQ_BF16) {
    u16x8 h;
#pragma unroll
    for (int i = 0; i < 8; ++i) h[i] = float_to_bf16(f[i]);
    r.q[0] = __builtin_bit_cast(u32x4, h);
  } else {
    r.q[0] = __builtin_bit_cast(u32x4, f32x4{f[0], f[1], f[2], f[3]});
    r.q[sizeof(r.q) / 16 - 1] = __builtin_bit_cast(u32x4, f32x4{f[4], f[5], f[6], f[7]});
  }
  return r;
}

// One wave per row; NP = packs of 8 elements each lane caches: cols <= 64 * 8 * NP and 8 | cols.
// A wave walks rows gw, gw + nwaves, ... and leaves the absmax over all of them in wave_absmax[gw].
// x, gamma and beta are all requested before anything is waited for and stay in registers in
// storage format (half the registers of fp32 for the 16-bit types), so the row's critical path
// holds one memory round trip, not two.
template<typename T, int NP, bool SKIP, bool EXACT>
__global__ void __launch_bounds__(kLnBlock)
ln_observer_wave_rows(const typename TT<T>::storage* __restrict__ x,
                      const typename TT<T>::storage* __restrict__ gamma,
                      const typename TT<T>::storage* __restrict__ beta,
                      typename TT<T>::storage* __restrict__ y, float* __restrict__ wave_absmax,
                      int64_t rows, int64_t cols, double eps64, SkipArgs<T> sk) {
  const float eps = (float)eps64;
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t gw = (int64_t)blockIdx.x * (kLnBlock / kWave) + (threadIdx.x >> 6);
  const int64_t nwaves = (int64_t)gridDim.x * (kLnBlock / kWave);
  const int npacks = (int)(cols / 8);
  float amax = 0.0f;
  RawPack<T> gr[NP], br[NP];
  bool first = true;
  for (int64_t row = gw; row < rows; row += nwaves) {
    const typename TT<T>::storage* xr = x + row * cols;
    typename TT<T>::storage* yr = y + row * cols;
    RawPack<T> v[NP];
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      const int p = lane + i * kWave;
      if (p < npacks) v[i] = load_raw<T>(xr + (int64_t)p * 8);
    }
    if (SKIP) {
      // the residual sum, rounded to T, takes the place of x in the registers
      RawPack<T> sr[NP], bb[NP];
#pragma unroll
      for (int i = 0; i < NP; ++i) {
        const int p = lane + i * kWave;
        if (p < npacks) {
          if (sk.skip) sr[i] = load_raw<T>(sk.skip + row * cols + (int64_t)p * 8);
          if (sk.bias) bb[i] = load_raw<T>(sk.bias + (int64_t)p * 8);
        }
      }
#pragma unroll
      for (int i = 0; i < NP; ++i) {
        const int p = lane + i * kWave;
        if (p < npacks) {
          float fx[8], fb[8], fs[8], o[8];
          widen<T>(v[i], fx);
#pragma unroll
          for (int e = 0; e < 8; ++e) fb[e] = fs[e] = 0.f;
          if (sk.bias) widen<T>(bb[i], fb);
          if (sk.skip) widen<T>(sr[i], fs);
#pragma unroll
          for (int e = 0; e < 8; ++e) o[e] = skip_sum<T>(fx[e], fb[e], fs[e], sk.alpha);
          v[i] = narrow<T>(o);
        }
      }
    }
    if (first) {
#pragma unroll
      for (int i = 0; i < NP; ++i) {
        const int p = lane + i * kWave;
        if (p < npacks) {
          if (gamma) gr[i] = load_raw<T>(gamma + (int64_t)p * 8);
          if (beta) br[i] = load_raw<T>(beta + (int64_t)p * 8);
        }
      }
      first = false;
    }
    float mean, inv;
    if constexpr (EXACT) {
      double sum64 = 0.0;
#pragma unroll
      for (int i = 0; i < NP; ++i) {
        const int p = lane + i * kWave;
        if (p < npacks) {
          float f[8];
          widen<T>(v[i], f);
#pragma unroll
          for (int e = 0; e < 8; ++e) sum64 += (double)f[e];
        }
      }
      sum64 = wave_reduce(sum64, OpSum());
      const double mean64 = sum64 / (double)cols;
      double q = 0.0;
#pragma unroll
      for (int i = 0; i < NP; ++i) {
        const int p = lane + i * kWave;
        if (p < npacks) {
          float f[8];
          widen<T>(v[i], f);
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const double d = (double)f[e] - mean64;
            q = __builtin_fma(d, d, q);
          }
        }
      }
      q = wave_reduce(q, OpSum());
      mean = (float)mean64;
      inv = exact_inv(q, (double)cols, eps64);
    } else {
      float sum = 0.0f;
#pragma unroll
      for (int i = 0; i < NP; ++i) {
        const int p = lane + i * kWave;
        if (p < npacks) {
          // (plain widen-and-add: a chain of v_dot2_f32_f16 on one accumulator came out of the
          // compiler with the same source register in every link)
          float f[8];
          widen<T>(v[i], f);
#pragma unroll
          for (int e = 0; e < 8; ++e) sum += f[e];
        }
      }
      sum = wave_reduce(sum, OpSum());
      mean = sum / (float)cols;
      float m2 = 0.0f;
#pragma unroll
      for (int i = 0; i < NP; ++i) {
        const int p = lane + i * kWave;
        if (p < npacks) {
          float f[8];
          widen<T>(v[i], f);
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float d = f[e] - mean;
            m2 = __builtin_fmaf(d, d, m2);
          }
        }
      }
      m2 = wave_reduce(m2, OpSum());
      const float var = fmaxf(m2 / (float)cols, 0.0f);
      inv = 1.0f / __builtin_sqrtf(var + eps);
    }
    f16x8 amax8 = {(f16)0.0f, (f16)0.0f, (f16)0.0f, (f16)0.0f, (f16)0.0f, (f16)0.0f, (f16)0.0f, (f16)0.0f};
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      const int p = lane + i * kWave;
      if (p < npacks) {
        if constexpr (TT<T>::dtype == OFQ_F16) {
          // the affine in T is native packed fp16 arithmetic: one rounding per multiply and per
          // add, which is what rounding the fp32 result of each step to fp16 gives as well
          float f[8];
          widen<T>(v[i], f);
          f16x8 t;
#pragma unroll
          for (int e = 0; e < 8; ++e) t[e] = (f16)((f[e] - mean) * inv);
          if (gamma) t = t * __builtin_bit_cast(f16x8, gr[i].q[0]);
          if (beta) t = t + __builtin_bit_cast(f16x8, br[i].q[0]);
          else if (gamma) t = t + (f16)0.0f;  // the reference adds its default beta 0: -0 -> +0
          amax8 = __builtin_elementwise_max(amax8, __builtin_elementwise_abs(t));
          *reinterpret_cast<u32x4*>(yr + (int64_t)p * 8) = __builtin_bit_cast(u32x4, t);
        } else {
          float f[8], g[8], b[8], o[8];
          widen<T>(v[i], f);
          if (gamma) widen<T>(gr[i], g);
          if (beta) widen<T>(br[i], b);
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            float t = normalised<T>(f[e] - mean, inv);
            if (gamma) t = TT<T>::round(t * g[e]);
            if (beta) t = TT<T>::round(t + b[e]);
            else if (gamma) t = t + 0.0f;  // default beta 0 of the reference: -0 -> +0
            o[e] = t;
            amax = fmaxf(amax, fabsf(t));
          }
          store8<T>(yr + (int64_t)p * 8, o);
        }
      }
    }
    if constexpr (TT<T>::dtype == OFQ_F16) {
#pragma unroll
      for (int e = 0; e < 8; ++e) amax = fmaxf(amax, (float)amax8[e]);
    }
  }
  amax = wave_reduce(amax, OpMax());
  if (lane == 0 && gw < rows) wave_absmax[gw] = amax;
}

// Rows of exactly 512 * NP elements of a 16-bit type, gamma and beta both present, no residual:
// the same one-wave-per-row scheme with nothing conditional inside the row (no partial packs, no
// null checks), the deviations kept in registers between the variance and the normalisation, the
// fp16 row sum formed with packed dot products, and, when a wave walks several rows (LOOP), the
// next row requested before the current one is worked on.  At 2048 x 4096 the general kernel
// spends about 1100 vector instructions per row, this one about half; both are bound by that
// arithmetic once the row has arrived, not by HBM.
// SKIP: the normalised row is (x + bias[c]) + skip * T(alpha) (see the top of the file), formed
// as the row arrives and kept in storage format in place of x; the next row is then not
// requested ahead (LOOP must be false), the registers hold the residual inputs instead.
template<typename T, int NP, bool LOOP, bool SKIP, bool EXACT>
__global__ void __launch_bounds__(kLnBlock)
ln_observer_wave_full(const typename TT<T>::storage* __restrict__ x,
                      const typename TT<T>::storage* __restrict__ gamma,
                      const typename TT<T>::storage* __restrict__ beta,
                      typename TT<T>::storage* __restrict__ y, float* __restrict__ wave_absmax,
                      int64_t rows, double eps64, SkipArgs<T> sk) {
  const float eps = (float)eps64;
  static_assert(sizeof(typename TT<T>::storage) == 2, "16-bit types only");
  static_assert(!(SKIP && LOOP), "the residual variant does not prefetch");
  constexpr int kCols = NP * 512;
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t gw = (int64_t)blockIdx.x * (kLnBlock / kWave) + (threadIdx.x >> 6);
  const int64_t nwaves = (int64_t)gridDim.x * (kLnBlock / kWave);
  if (gw >= rows) return;
  u32x4 cur[NP], nxt[LOOP ? NP : 1], gr[NP], br[NP];
  {
    const typename TT<T>::storage* xr = x + gw * kCols + lane * 8;
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      cur[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xr + i * 512));
    }
  }
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    gr[i] = *reinterpret_cast<const u32x4*>(gamma + lane * 8 + i * 512);
    br[i] = *reinterpret_cast<const u32x4*>(beta + lane * 8 + i * 512);
  }
  float amax = 0.0f;
  f16x8 amax8 = {(f16)0.0f, (f16)0.0f, (f16)0.0f, (f16)0.0f, (f16)0.0f, (f16)0.0f, (f16)0.0f, (f16)0.0f};
  for (int64_t row = gw; row < rows; row += nwaves) {
    bool more = false;
    if constexpr (LOOP) {
      more = row + nwaves < rows;  // the same for every lane
      if (more) {
        const typename TT<T>::storage* xn = x + (row + nwaves) * kCols + lane * 8;
#pragma unroll
        for (int i = 0; i < NP; ++i) {
          nxt[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xn + i * 512));
        }
      }
    }
    if constexpr (SKIP) {
      if (row != gw) {  // (rows after the wave's first: x was not requested ahead)
        const typename TT<T>::storage* xr2 = x + row * kCols + lane * 8;
#pragma unroll
        for (int i = 0; i < NP; ++i) {
          cur[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xr2 + i * 512));
        }
      }
      u32x4 sr[NP], bb[NP];
#pragma unroll
      for (int i = 0; i < NP; ++i) {
        if (sk.skip) {
          sr[i] = __builtin_nontemporal_load(
              reinterpret_cast<const u32x4*>(sk.skip + row * kCols + lane * 8 + i * 512));
        }
        if (sk.bias) bb[i] = *reinterpret_cast<const u32x4*>(sk.bias + lane * 8 + i * 512);
      }
#pragma unroll
      for (int i = 0; i < NP; ++i) {
        if constexpr (TT<T>::dtype == OFQ_F16) {
          // native packed fp16 arithmetic rounds once per operation, which is what rounding the
          // fp32 result of each operation to fp16 gives as well (an absent input enters as +0)
          f16x8 v = __builtin_bit_cast(f16x8, cur[i]);
          const f16x8 zero8 = {(f16)0.0f, (f16)0.0f, (f16)0.0f, (f16)0.0f, (f16)0.0f, (f16)0.0f, (f16)0.0f, (f16)0.0f};
          v = v + (sk.bias ? __builtin_bit_cast(f16x8, bb[i]) : zero8);
          const f16 a = (f16)sk.alpha;
          const f16x8 sa = sk.skip ? __builtin_bit_cast(f16x8, sr[i]) * a : zero8 * a;
          v = v + sa;
          cur[i] = __builtin_bit_cast(u32x4, v);
        } else {
          RawPack<T> xp, sp, bp;
          xp.q[0] = cur[i];
          float fx[8], fb[8], fs[8], o[8];
          widen<T>(xp, fx);
#pragma unroll
          for (int e = 0; e < 8; ++e) fb[e] = fs[e] = 0.f;
          if (sk.bias) { bp.q[0] = bb[i]; widen<T>(bp, fb); }
          if (sk.skip) { sp.q[0] = sr[i]; widen<T>(sp, fs); }
#pragma unroll
          for (int e = 0; e < 8; ++e) o[e] = skip_sum<T>(fx[e], fb[e], fs[e], sk.alpha);
          cur[i] = narrow<T>(o).q[0];
        }
      }
    }
    float f[NP][8];
    float sum = 0.0f;
    double sum64 = 0.0;
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      RawPack<T> rp;
      rp.q[0] = cur[i];
      widen<T>(rp, f[i]);
      if constexpr (EXACT) {
#pragma unroll
        for (int e = 0; e < 8; ++e) sum64 += (double)f[i][e];
      } else if constexpr (TT<T>::dtype == OFQ_F16) {
        // (1, 1) held in a register: with the constant as a literal operand the compiler emits
        // the four dot products of a pack with one and the same source register
        uint32_t ones_bits = 0x3c003c00u;
        asm volatile("" : "+v"(ones_bits));
        const f16x2 ones = __builtin_bit_cast(f16x2, ones_bits);
        // (pairs taken from the whole-vector bit cast: `bit_cast<f16x2>(cur[i][w])` came out of
        // the compiler as word 0 for every w)
        const f16x8 h = __builtin_bit_cast(f16x8, cur[i]);
        sum = __builtin_amdgcn_fdot2(__builtin_shufflevector(h, h, 0, 1), ones, sum, false);
        sum = __builtin_amdgcn_fdot2(__builtin_shufflevector(h, h, 2, 3), ones, sum, false);
        sum = __builtin_amdgcn_fdot2(__builtin_shufflevector(h, h, 4, 5), ones, sum, false);
        sum = __builtin_amdgcn_fdot2(__builtin_shufflevector(h, h, 6, 7), ones, sum, false);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) sum += f[i][e];
      }
    }
    float mean, inv;
    if constexpr (EXACT) {
      sum64 = wave_reduce(sum64, OpSum());
      const double mean64 = sum64 / (double)kCols;
      mean = (float)mean64;
      double q = 0.0;
#pragma unroll
      for (int i = 0; i < NP; ++i) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const double d = (double)f[i][e] - mean64;
          q = __builtin_fma(d, d, q);
          f[i][e] = f[i][e] - mean;
        }
      }
      q = wave_reduce(q, OpSum());
      inv = exact_inv(q, (double)kCols, eps64);
    } else {
      sum = wave_reduce(sum, OpSum());
      mean = sum / (float)kCols;
      float m2 = 0.0f;
#pragma unroll
      for (int i = 0; i < NP; ++i) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          f[i][e] = f[i][e] - mean;
          m2 = __builtin_fmaf(f[i][e], f[i][e], m2);
        }
      }
      m2 = wave_reduce(m2, OpSum());
      const float var = fmaxf(m2 / (float)kCols, 0.0f);
      inv = 1.0f / __builtin_sqrtf(var + eps);
    }
    typename TT<T>::storage* yr = y + row * kCols + lane * 8;
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      if constexpr (TT<T>::dtype == OFQ_F16) {
        f16x8 t;
#pragma unroll
        for (int e = 0; e < 8; ++e) t[e] = (f16)(f[i][e] * inv);
        t = t * __builtin_bit_cast(f16x8, gr[i]);
        t = t + __builtin_bit_cast(f16x8, br[i]);
        // |t| by clearing the sign bits of the four words (elementwise abs of the vector comes
        // out as three instructions per pair)
        const u32x4 tb = __builtin_bit_cast(u32x4, t);
        const u32x4 ab = {tb[0] & 0x7FFF7FFFu, tb[1] & 0x7FFF7FFFu, tb[2] & 0x7FFF7FFFu,
                          tb[3] & 0x7FFF7FFFu};
        amax8 = __builtin_elementwise_max(amax8, __builtin_bit_cast(f16x8, ab));
        *reinterpret_cast<u32x4*>(yr + i * 512) = tb;
      } else {
        RawPack<T> gp, bp;
        gp.q[0] = gr[i];
        bp.q[0] = br[i];
        float g[8], b[8], o[8];
        widen<T>(gp, g);
        widen<T>(bp, b);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float t = normalised<T>(f[i][e], inv);
          t = TT<T>::round(t * g[e]);
          t = TT<T>::round(t + b[e]);
          o[e] = t;
          amax = fmaxf(amax, fabsf(t));
        }
        store8<T>(yr + i * 512, o);
      }
    }
    if constexpr (LOOP) {
      if (more) {
#pragma unroll
        for (int i = 0; i < NP; ++i) cur[i] = nxt[i];
      }
    }
  }
  if constexpr (TT<T>::dtype == OFQ_F16) {
#pragma unroll
    for (int e = 0; e < 8; ++e) amax = fmaxf(amax, (float)amax8[e]);
  }
  amax = wave_reduce(amax, OpMax());
  if (lane == 0) wave_absmax[gw] = amax;
}

// any cols: three passes over the row through L2 (the row was just read, so only the first
// pass touches HBM), scalar accesses.
template<typename T, bool SKIP, bool EXACT>
__global__ void __launch_bounds__(kLnBlock)
ln_observer_rows_generic(const typename TT<T>::storage* __restrict__ x,
                         const typename TT<T>::storage* __restrict__ gamma,
                         const typename TT<T>::storage* __restrict__ beta,
                         typename TT<T>::storage* __restrict__ y, float* __restrict__ row_absmax,
                         int64_t cols, double eps64, SkipArgs<T> sk) {
  __shared__ float smem[kLnBlock / kWave];
  __shared__ double smem64[EXACT ? kLnBlock / kWave : 1];
  const float eps = (float)eps64;
  const int64_t row = blockIdx.x;
  const typename TT<T>::storage* xr = x + row * cols;
  typename TT<T>::storage* yr = y + row * cols;
  auto input = [&](int64_t c) {
    const float xv = TT<T>::load(xr + c);
    if (!SKIP) return xv;
    const float bv = sk.bias ? TT<T>::load(sk.bias + c) : 0.f;
    const float sv = sk.skip ? TT<T>::load(sk.skip + row * cols + c) : 0.f;
    return skip_sum<T>(xv, bv, sv, sk.alpha);
  };
  float mean, inv;
  if constexpr (EXACT) {
    double sum64 = 0.0;
    for (int64_t c = threadIdx.x; c < cols; c += kLnBlock) sum64 += (double)input(c);
    sum64 = block_reduce(sum64, OpSum(), smem64);
    const double mean64 = sum64 / (double)cols;
    double q = 0.0;
    for (int64_t c = threadIdx.x; c < cols; c += kLnBlock) {
      const double d = (double)input(c) - mean64;
      q = __builtin_fma(d, d, q);
    }
    q = block_reduce(q, OpSum(), smem64);
    mean = (float)mean64;
    inv = exact_inv(q, (double)cols, eps64);
  } else {
    float sum = 0.0f;
    for (int64_t c = threadIdx.x; c < cols; c += kLnBlock) sum += input(c);
    sum = block_reduce(sum, OpSum(), smem);
    mean = sum / (float)cols;
    float m2 = 0.0f;
    for (int64_t c = threadIdx.x; c < cols; c += kLnBlock) {
      const float d = input(c) - mean;
      m2 = __builtin_fmaf(d, d, m2);
    }
    m2 = block_reduce(m2, OpSum(), smem);
    const float var = fmaxf(m2 / (float)cols, 0.0f);
    inv = 1.0f / __builtin_sqrtf(var + eps);
  }
  float amax = 0.0f;
  for (int64_t c = threadIdx.x; c < cols; c += kLnBlock) {
    float t = normalised<T>(input(c) - mean, inv);
    if (gamma) t = TT<T>::round(t * TT<T>::load(gamma + c));
    if (beta) t = TT<T>::round(t + TT<T>::load(beta + c));
    else if (gamma) t = t + 0.0f;  // default beta 0 of the reference: -0 -> +0
    TT<T>::store(yr + c, t);
    amax = fmaxf(amax, fabsf(t));
  }
  amax = block_reduce(amax, OpMax(), smem);
  if (threadIdx.x == 0) row_absmax[row] = amax;
}

// one wave folds the n partial maxima
__global__ void __launch_bounds__(kWave)
ln_observer_finalize(const float* __restrict__ part, int64_t n, int bits,
                     float* __restrict__ scale, float* __restrict__ zero_point) {
  float amax = 0.0f;
  const int64_t n4 = (reinterpret_cast<uintptr_t>(part) & 15u) == 0 ? n / 4 : 0;
  const f32x4* p4 = reinterpret_cast<const f32x4*>(part);
  for (int64_t i = threadIdx.x; i < n4; i += kWave) {
    const f32x4 q = p4[i];
    amax = fmaxf(fmaxf(amax, fmaxf(q[0], q[1])), fmaxf(q[2], q[3]));
  }
  for (int64_t i = n4 * 4 + threadIdx.x; i < n; i += kWave) amax = fmaxf(amax, part[i]);
  amax = wave_reduce(amax, OpMax());
  if (threadIdx.x == 0) {
    const float denominator = (float)(1 << (bits - 1)) - 1.0f;
    *scale = amax / denominator;
    *zero_point = 0.0f;
  }
}

// ---------------------------------------------------------------------------------------------
// LayerNorm -> observer -> int8 codes without the normalised tensor ever reaching memory
// (ofq_fused_layer_norm_quantization).  fp16 rows of exactly 512 * NP elements with gamma and beta.
// Two kernels:
//   first : the row kernel above without its store: a wave normalises its rows in registers,
//           keeps (mean, inv) of every row and the largest |y| it has seen;
//   second: every block folds the partial maxima into the scale (the arithmetic of
//           ln_observer_finalize, so every block gets the same bits), then a wave reads its rows
//           again -- from L2 where the first kernel left them: the same wave of the same block
//           took them there --, forms y with the stored statistics exactly as the first kernel
//           did, and quantises it the way quantize_half_to_bytes_kernel does.
// The codes are those of fused_layer_norm_min_max_observer followed by quantization (symmetric,
// per layer) of its y, bit for bit; traffic is x once from HBM, x once more from L2 and the codes
// (25 MB at 2048 x 4096 where the two ops move 58.7 MB).
// ---------------------------------------------------------------------------------------------
constexpr int kLnqBlock = 512;  // 8 waves: one copy of gamma and beta in LDS serves 8 rows

// gamma and beta of a block: fetched once (wave w fetches pack w of each), parked in LDS, read
// from there pack by pack.  Every wave of the block holding its own copy in registers cost 16 of
// a wave's 24 requests and as much traffic between L2 and the CU as x itself.
template<int NP>
struct LnRowF16 {
  u32x4 graw, braw;
  __device__ __forceinline__ void request(const uint16_t* gamma, const uint16_t* beta, int wave,
                                          int lane) {
    if (wave < NP) {  // the same for every lane of a wave
      graw = *reinterpret_cast<const u32x4*>(gamma + lane * 8 + wave * 512);
      braw = *reinterpret_cast<const u32x4*>(beta + lane * 8 + wave * 512);
    }
  }
  // [gamma NP x 64 pieces][beta NP x 64 pieces]; a barrier must follow before out() is used
  __device__ __forceinline__ void park(u32x4* lds, int wave, int lane) const {
    if (wave < NP) {
      lds[wave * 64 + lane] = graw;
      lds[(NP + wave) * 64 + lane] = braw;
    }
  }
  // y of pack i from the deviations d[8] = x - mean: T(d * inv), * gamma, + beta, each rounded to T
  __device__ __forceinline__ f16x8 out(const float* d, float inv, int i, const u32x4* lds,
                                       int lane) const {
    f16x8 t;
#pragma unroll
    for (int e = 0; e < 8; ++e) t[e] = (f16)normalised<f16>(d[e], inv);
    t = t * __builtin_bit_cast(f16x8, lds[i * 64 + lane]);
    t = t + __builtin_bit_cast(f16x8, lds[(NP + i) * 64 + lane]);
    return t;
  }
};

template<int NP, bool EXACT>
__global__ void __launch_bounds__(kLnqBlock)
ln_quant_first(const uint16_t* __restrict__ x, const uint16_t* __restrict__ gamma,
               const uint16_t* __restrict__ beta, float* __restrict__ block_absmax,
               float* __restrict__ stats, int64_t rows, double eps64) {
  constexpr int kCols = NP * 512;
  constexpr int kWaves = kLnqBlock / kWave;
  __shared__ float wmax[kWaves];
  __shared__ u32x4 params[2 * NP * 64];
  const float eps = (float)eps64;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t gw = (int64_t)blockIdx.x * kWaves + wave;
  const int64_t nwaves = (int64_t)gridDim.x * kWaves;
  LnRowF16<NP> prm;
  prm.request(gamma, beta, wave, lane);
  u32x4 cur[NP];
  {
    // (a wave past the last row re-reads row 0 and skips the loop: it only joins the barriers)
    const uint16_t* xr = x + (gw < rows ? gw : 0) * kCols + lane * 8;
#pragma unroll
    for (int i = 0; i < NP; ++i) cur[i] = *reinterpret_cast<const u32x4*>(xr + i * 512);
  }
  prm.park(params, wave, lane);
  __syncthreads();
  f16x8 amax8 = {(f16)0.0f, (f16)0.0f, (f16)0.0f, (f16)0.0f, (f16)0.0f, (f16)0.0f, (f16)0.0f, (f16)0.0f};
  for (int64_t row = gw; row < rows; row += nwaves) {
    if (row != gw) {
      const uint16_t* xr = x + row * kCols + lane * 8;
#pragma unroll
      for (int i = 0; i < NP; ++i) cur[i] = *reinterpret_cast<const u32x4*>(xr + i * 512);
    }
    float f[NP][8];
    float sum = 0.0f;
    double sum64 = 0.0;
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      RawPack<f16> rp;
      rp.q[0] = cur[i];
      widen<f16>(rp, f[i]);
      if constexpr (EXACT) {
#pragma unroll
        for (int e = 0; e < 8; ++e) sum64 += (double)f[i][e];
      } else {
        uint32_t ones_bits = 0x3c003c00u;  // (1, 1) held in a register, see ln_observer_wave_full
        asm volatile("" : "+v"(ones_bits));
        const f16x2 ones = __builtin_bit_cast(f16x2, ones_bits);
        const f16x8 h = __builtin_bit_cast(f16x8, cur[i]);
        sum = __builtin_amdgcn_fdot2(__builtin_shufflevector(h, h, 0, 1), ones, sum, false);
        sum = __builtin_amdgcn_fdot2(__builtin_shufflevector(h, h, 2, 3), ones, sum, false);
        sum = __builtin_amdgcn_fdot2(__builtin_shufflevector(h, h, 4, 5), ones, sum, false);
        sum = __builtin_amdgcn_fdot2(__builtin_shufflevector(h, h, 6, 7), ones, sum, false);
      }
    }
    float mean, inv;
    if constexpr (EXACT) {
      sum64 = wave_reduce(sum64, OpSum());
      const double mean64 = sum64 / (double)kCols;
      mean = (float)mean64;
      double q = 0.0;
#pragma unroll
      for (int i = 0; i < NP; ++i) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const double d = (double)f[i][e] - mean64;
          q = __builtin_fma(d, d, q);
          f[i][e] = f[i][e] - mean;
        }
      }
      q = wave_reduce(q, OpSum());
      inv = exact_inv(q, (double)kCols, eps64);
    } else {
      sum = wave_reduce(sum, OpSum());
      mean = sum / (float)kCols;
      float m2 = 0.0f;
#pragma unroll
      for (int i = 0; i < NP; ++i) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          f[i][e] = f[i][e] - mean;
          m2 = __builtin_fmaf(f[i][e], f[i][e], m2);
        }
      }
      m2 = wave_reduce(m2, OpSum());
      const float var = fmaxf(m2 / (float)kCols, 0.0f);
      inv = 1.0f / __builtin_sqrtf(var + eps);
    }
    if (lane == 0) {
      stats[2 * row] = mean;
      stats[2 * row + 1] = inv;
    }
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      const u32x4 tb = __builtin_bit_cast(u32x4, prm.out(f[i], inv, i, params, lane));
      const u32x4 ab = {tb[0] & 0x7FFF7FFFu, tb[1] & 0x7FFF7FFFu, tb[2] & 0x7FFF7FFFu,
                        tb[3] & 0x7FFF7FFFu};
      amax8 = __builtin_elementwise_max(amax8, __builtin_bit_cast(f16x8, ab));
    }
  }
  float amax = 0.0f;
#pragma unroll
  for (int e = 0; e < 8; ++e) amax = fmaxf(amax, (float)amax8[e]);
  amax = wave_reduce(amax, OpMax());
  // one partial maximum per block, so that the second kernel folds them with one request
  if (lane == 0) wmax[wave] = amax;
  __syncthreads();
  if (threadIdx.x == 0) {
    amax = wmax[0];
#pragma unroll
    for (int wv = 1; wv < kWaves; ++wv) amax = fmaxf(amax, wmax[wv]);
    block_absmax[blockIdx.x] = amax;
  }
}

// SPLIT: a row is taken by SPLIT waves of SPLIT different blocks, NP / SPLIT packs each (nothing
// in this kernel crosses the lanes of a row), so that few rows still make enough waves to
// overlap one wave's arithmetic with another's requests.  Block b works on the rows of block
// p = (b / (8 * SPLIT)) * 8 + b % 8 of the first kernel, part (b / 8) % SPLIT: b and p agree
// modulo 8, the number of XCDs the blocks are dealt over, so a row is read again through the L2
// that holds it.  The grid is ceil(first_grid / 8) * 8 * SPLIT blocks.
template<int NP, int SPLIT>
__global__ void __launch_bounds__(kLnqBlock)
ln_quant_second(const uint16_t* __restrict__ x, const uint16_t* __restrict__ gamma,
                const uint16_t* __restrict__ beta, const float* __restrict__ part, int64_t nparts,
                const float* __restrict__ stats, int8_t* __restrict__ codes,
                float* __restrict__ scale, float* __restrict__ zero_point, int64_t rows, int bits,
                int first_grid) {
  static_assert(NP % SPLIT == 0, "whole packs per part");
  constexpr int kCols = NP * 512;
  constexpr int NPW = NP / SPLIT;  // packs of a row this wave takes
  constexpr int kWaves = kLnqBlock / kWave;
  __shared__ float wmax[kWaves];
  __shared__ u32x4 params[2 * NPW * 64];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t fb = ((int64_t)blockIdx.x / (8 * SPLIT)) * 8 + blockIdx.x % 8;
  const int part_of_row = (int)((blockIdx.x / 8) % SPLIT);
  const int pack0 = part_of_row * NPW;
  const int64_t gw = fb * kWaves + wave;
  const int64_t nwaves = (int64_t)first_grid * kWaves;
  const bool active = gw < rows;
  // Requests in the order of their use: the partial maxima (one 16-byte piece per thread:
  // nparts <= 512 <= 4 * kLnqBlock), the statistics of the wave's first row, the wave's share of
  // the parameters, then the row, so that the maxima can be folded and the parameters parked
  // while the row is still on its way.
  const int64_t n4 = (nparts + 3) / 4;
  const int64_t pidx = (int64_t)threadIdx.x < n4 ? threadIdx.x : 0;
  f32x4 pq = reinterpret_cast<const f32x4*>(part)[pidx];
  const float* st0 = stats + 2 * (active ? gw : 0);
  float mean0 = st0[0], inv0 = st0[1];
  LnRowF16<NPW> prm;
  prm.request(gamma + pack0 * 512, beta + pack0 * 512, wave, lane);
  u32x4 cur[NPW];
  {
    const uint16_t* xr = x + (active ? gw : 0) * kCols + pack0 * 512 + lane * 8;
#pragma unroll
    for (int i = 0; i < NPW; ++i) cur[i] = *reinterpret_cast<const u32x4*>(xr + i * 512);
  }
  prm.park(params, wave, lane);
  // scale = max of the partial maxima / (2^(bits-1) - 1), the same operations in every block
  // (the last piece may reach up to three floats past the partials: masked)
  float amax = 0.0f;
  {
#pragma unroll
    for (int e = 0; e < 4; ++e) amax = fmaxf(amax, pidx * 4 + e < nparts ? pq[e] : 0.0f);
    amax = wave_reduce(amax, OpMax());
    if (lane == 0) wmax[wave] = amax;
    __syncthreads();  // (also orders the parked parameters before their use)
    amax = 0.0f;
#pragma unroll
    for (int wv = 0; wv < kWaves; ++wv) amax = fmaxf(amax, wmax[wv]);
  }
  const float upper = (float)(1 << (bits - 1)) - 1.0f;
  const float s = amax / upper;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *scale = s;
    *zero_point = 0.0f;
  }
  if (!active) return;
  // quantisation of quantize_half_to_bytes_kernel, symmetric scheme
  const float mag = __builtin_fabsf(s);
  const bool recip_ok = mag >= 0x1p-60f && mag <= 0x1p60f;
  const float recip = recip_ok ? 1.0f / s : 0.f;
  const int hi = (int)upper, lo = -hi - 1;
  // (the branch on the scale's range is taken once per wave: inside the loop both quotients
  // would be computed for every element and one of them selected)
  auto walk = [&](auto fast) {
    for (int64_t row = gw; row < rows; row += nwaves) {
      if (row != gw) {
        const uint16_t* xr = x + row * kCols + pack0 * 512 + lane * 8;
#pragma unroll
        for (int i = 0; i < NPW; ++i) cur[i] = *reinterpret_cast<const u32x4*>(xr + i * 512);
      }
      float mean = mean0, inv = inv0;
      if (row != gw) {
        mean = stats[2 * row];
        inv = stats[2 * row + 1];
      }
      int8_t* cr = codes + row * kCols + pack0 * 512 + lane * 8;
#pragma unroll
      for (int i = 0; i < NPW; ++i) {
        RawPack<f16> rp;
        rp.q[0] = cur[i];
        float d[8];
        widen<f16>(rp, d);
#pragma unroll
        for (int e = 0; e < 8; ++e) d[e] = d[e] - mean;
        // (held as four packed registers: otherwise the affine is emitted element by element)
        u32x4 yb = __builtin_bit_cast(u32x4, prm.out(d, inv, i, params, lane));
        asm volatile("" : "+v"(yb[0]), "+v"(yb[1]), "+v"(yb[2]), "+v"(yb[3]));
        const f16x8 y = __builtin_bit_cast(f16x8, yb);
        uint32_t words[2];
#pragma unroll
        for (int e4 = 0; e4 < 8; e4 += 4) {
          uint32_t b[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float v = (float)y[e4 + j];
            float q;
            if constexpr (decltype(fast)::value) {
              // (y is finite here: an infinite y makes the scale infinite, which is the other
              // branch)
              q = div_of_finite_half_value(v, s, recip);
            } else {
              q = v / s;
            }
            const float t = __builtin_rintf(q);
            int c;
            asm("v_cvt_i32_f32 %0, %1" : "=v"(c) : "v"(t));  // saturates; NaN -> 0
            b[j] = (uint32_t)clamp_i32(c, lo, hi);
          }
          const uint32_t lo2 = __builtin_amdgcn_perm(b[1], b[0], 0x0c0c0400u);
          const uint32_t hi2 = __builtin_amdgcn_perm(b[3], b[2], 0x04000c0cu);
          words[e4 / 4] = lo2 | hi2;
        }
        const u32x2 w2 = {words[0], words[1]};
        __builtin_nontemporal_store(w2, reinterpret_cast<u32x2*>(cr + i * 512));
      }
    }
  };
  if (recip_ok) {
    walk(std::true_type());
  } else {
    walk(std::false_type());
  }
}

// host-side rounding of a float to T (round to nearest even)
template<typename T>
float round_to_T_host(float v) {
  if (TT<T>::dtype == OFQ_F16) return (float)(_Float16)v;
  if (TT<T>::dtype == OFQ_BF16) {
    uint32_t u;
    __builtin_memcpy(&u, &v, 4);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return v;  // NaN stays NaN
    u += 0x7FFFu + ((u >> 16) & 1u);
    u &= 0xFFFF0000u;
    __builtin_memcpy(&v, &u, 4);
    return v;
  }
  return v;
}

template<typename T, bool SKIP, bool EXACT>
int launch(hipStream_t st, const void* x, const void* gamma, const void* beta, void* y,
           float* scale, float* zero_point, int64_t rows, int64_t cols, double eps, int bits,
           float* ws, const void* bias, const void* skip, double alpha) {
  typedef typename TT<T>::storage S;
  const S* xs = static_cast<const S*>(x);
  const S* gs = static_cast<const S*>(gamma);
  const S* bs = static_cast<const S*>(beta);
  S* ys = static_cast<S*>(y);
  SkipArgs<T> sk;
  sk.bias = static_cast<const S*>(bias);
  sk.skip = static_cast<const S*>(skip);
  // T(alpha): the reference casts its float alpha to T (skip_layer_norm_kernel.cu:36,62)
  sk.alpha = round_to_T_host<T>((float)alpha);
  const bool vec_ok = cols % 8 == 0 && ofq_aligned16(x) && ofq_aligned16(y)
                      && ofq_aligned16(gamma) && ofq_aligned16(beta) && ofq_aligned16(bias)
                      && ofq_aligned16(skip) && (cols * sizeof(S)) % 16 == 0;
  const int64_t npacks = cols / 8;
  int64_t nparts = rows;
  constexpr int kWavesPerBlock = kLnBlock / kWave;
  // fp32 rows beyond 2048 elements would not fit a lane's registers at two waves per SIMD
  const int64_t wave_packs = (sizeof(S) == 4 ? 4 : 8) * kWave;
  if constexpr (sizeof(S) == 2) {
    const int np = (int)(cols / 512);
    if (vec_ok && gamma != nullptr && beta != nullptr && cols % 512 == 0
        && (np == 1 || np == 2 || np == 4 || np == 8)) {
      // one row per wave while the rows fit 16 waves per CU; beyond that 8 waves per CU walk the
      // rows with the next row in flight
      const bool loop = rows > 256 * 16;
      // (the residual variant at NP = 8 holds 230 registers: 8 waves per CU there as well)
      const int64_t waves = loop ? 256 * 8 : rows;
      const int grid = (int)((waves + kWavesPerBlock - 1) / kWavesPerBlock);
      nparts = waves;
#define OFQ_LN_FULL(NPV)                                                                        \
  if (SKIP) {                                                                                    \
    ln_observer_wave_full<T, NPV, false, SKIP, EXACT><<<grid, kLnBlock, 0, st>>>(                \
        xs, gs, bs, ys, ws, rows, eps, sk);                                                      \
  } else if (loop) {                                                                             \
    ln_observer_wave_full<T, NPV, true, false, EXACT><<<grid, kLnBlock, 0, st>>>(                \
        xs, gs, bs, ys, ws, rows, eps, sk);                                                      \
  } else {                                                                                       \
    ln_observer_wave_full<T, NPV, false, false, EXACT><<<grid, kLnBlock, 0, st>>>(               \
        xs, gs, bs, ys, ws, rows, eps, sk);                                                      \
  }
      switch (np) {
        case 1: OFQ_LN_FULL(1) break;
        case 2: OFQ_LN_FULL(2) break;
        case 4: OFQ_LN_FULL(4) break;
        default: OFQ_LN_FULL(8) break;
      }
#undef OFQ_LN_FULL
      ln_observer_finalize<<<1, kWave, 0, st>>>(ws, nparts, bits, scale, zero_point);
      return ofq_check_launch();
    }
  }
  if (vec_ok && npacks <= wave_packs) {
    // about 32 KB of rows in flight per CU streams best: 4 waves per CU for 8 KB rows, up to 16
    // for rows of 2 KB and less (16384 x 1024 fp16: 33 -> 23 us); with more rows than waves a
    // wave walks several rows and the waves of a CU drift apart
    const int64_t row_bytes = cols * (int64_t)sizeof(S);
    int64_t per_cu = 32768 / row_bytes;
    per_cu = per_cu < 4 ? 4 : (per_cu > 16 ? 16 : per_cu);
    const int64_t wcap = 256 * per_cu;
    const int64_t waves = rows < wcap ? rows : wcap;
    const int grid = (int)((waves + kWavesPerBlock - 1) / kWavesPerBlock);
    nparts = (int64_t)grid * kWavesPerBlock < rows ? (int64_t)grid * kWavesPerBlock : rows;
#define OFQ_LN_WAVE(NPV)                                                                       \
  ln_observer_wave_rows<T, NPV, SKIP, EXACT><<<grid, kLnBlock, 0, st>>>(xs, gs, bs, ys, ws, rows, \
                                                                        cols, eps, sk)
    if (npacks <= kWave) {
      OFQ_LN_WAVE(1);
    } else if (npacks <= 2 * kWave) {
      OFQ_LN_WAVE(2);
    } else if (npacks <= 4 * kWave) {
      OFQ_LN_WAVE(4);
    } else {
      OFQ_LN_WAVE(8);
    }
#undef OFQ_LN_WAVE
  } else if (vec_ok && npacks <= kLnBlock) {
    ln_observer_rows<T, 1, SKIP, EXACT><<<(int)rows, kLnBlock, 0, st>>>(xs, gs, bs, ys, ws, cols, eps, sk);
  } else if (vec_ok && npacks <= 2 * kLnBlock) {
    ln_observer_rows<T, 2, SKIP, EXACT><<<(int)rows, kLnBlock, 0, st>>>(xs, gs, bs, ys, ws, cols, eps, sk);
  } else if (vec_ok && npacks <= 4 * kLnBlock) {
    ln_observer_rows<T, 4, SKIP, EXACT><<<(int)rows, kLnBlock, 0, st>>>(xs, gs, bs, ys, ws, cols, eps, sk);
  } else if (vec_ok && npacks <= 8 * kLnBlock) {
    ln_observer_rows<T, 8, SKIP, EXACT><<<(int)rows, kLnBlock, 0, st>>>(xs, gs, bs, ys, ws, cols, eps, sk);
  } else {
    ln_observer_rows_generic<T, SKIP, EXACT><<<(int)rows, kLnBlock, 0, st>>>(xs, gs, bs, ys, ws, cols,
                                                                      eps, sk);
  }
  ln_observer_finalize<<<1, kWave, 0, st>>>(ws, nparts, bits, scale, zero_point);
  return ofq_check_launch();
}

int run(void* stream, const void* x, const void* bias, const void* skip, double alpha,
        bool with_skip, const void* gamma, const void* beta, void* y, float* scale,
        float* zero_point, int t_dtype, int64_t rows, int64_t cols, double epsilon,
        int quantization_bit, int statistics, void* workspace, size_t workspace_bytes) {
  OFQ_RETURN_IF(quantization_bit <= 1 || quantization_bit > 8, OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(statistics != OFQ_LN_STATS_FP32 && statistics != OFQ_LN_STATS_FP64,
                OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(t_dtype != OFQ_F16 && t_dtype != OFQ_BF16 && t_dtype != OFQ_F32,
                OFQ_ERR_BAD_DTYPE);
  OFQ_RETURN_IF(rows < 1 || cols < 1 || rows > 0x7FFFFFFF, OFQ_ERR_BAD_SHAPE);
  OFQ_RETURN_IF(x == nullptr || y == nullptr || scale == nullptr || zero_point == nullptr,
                OFQ_ERR_NULL_POINTER);
  OFQ_RETURN_IF(workspace == nullptr || workspace_bytes < (size_t)rows * sizeof(float),
                OFQ_ERR_WORKSPACE);
  hipStream_t st = static_cast<hipStream_t>(stream);
  float* ws = static_cast<float*>(workspace);
  const double eps = epsilon;  // (the fp32 statistics round it to fp32 in the kernel)
#define OFQ_LN_RUN2(T, EX)                                                                     \
  return with_skip ? launch<T, true, EX>(st, x, gamma, beta, y, scale, zero_point, rows, cols, \
                                         eps, quantization_bit, ws, bias, skip, alpha)         \
                   : launch<T, false, EX>(st, x, gamma, beta, y, scale, zero_point, rows,      \
                                          cols, eps, quantization_bit, ws, nullptr, nullptr, 0.0)
#define OFQ_LN_RUN(T)                                    \
  if (statistics == OFQ_LN_STATS_FP64) OFQ_LN_RUN2(T, true); \
  OFQ_LN_RUN2(T, false)
  switch (t_dtype) {
    case OFQ_F16: OFQ_LN_RUN(f16);
    case OFQ_BF16: OFQ_LN_RUN(bf16);
    default: OFQ_LN_RUN(float);
  }
#undef OFQ_LN_RUN
#undef OFQ_LN_RUN2
}

// device address of `scratch` on the current device, looked up once per device
constexpr int kMaxDevices = 64;
std::atomic<float*> scratch_on_device[kMaxDevices];

int static_scratch(float** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return OFQ_ERR_LAUNCH;
  float* p = scratch_on_device[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    void* addr = nullptr;
    if (hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch)) != hipSuccess || addr == nullptr) {
      return OFQ_ERR_LAUNCH;
    }
    p = static_cast<float*>(addr);
    scratch_on_device[dev].store(p, std::memory_order_release);  // same value from any thread
  }
  *out = p;
  return OFQ_OK;
}

}  // namespace
}  // namespace ofq

extern "C" int ofq_fused_layer_norm_min_max_observer_static(void* stream, const void* x,
                                                            const void* gamma, const void* beta,
                                                            void* y, float* scale,
                                                            float* zero_point, int t_dtype,
                                                            int64_t rows, int64_t cols,
                                                            double epsilon, int quantization_bit) {
  if (rows > OFQ_LN_STATIC_MAX_ROWS) return OFQ_ERR_TOO_LARGE;
  float* ws = nullptr;
  const int st = ofq::static_scratch(&ws);
  if (st != OFQ_OK) return st;
  // every partial the finalize kernel reads is written by the row kernel of the same call, so
  // nothing has to be cleared between calls
  return ofq::run(stream, x, nullptr, nullptr, 0.0, false, gamma, beta, y, scale, zero_point,
                  t_dtype, rows, cols, epsilon, quantization_bit, OFQ_LN_STATS_FP32, ws,
                  (size_t)OFQ_LN_STATIC_MAX_ROWS * sizeof(float));
}

extern "C" size_t ofq_fused_layer_norm_min_max_observer_workspace_bytes(int, int64_t rows,
                                                                        int64_t) {
  return rows > 0 ? (size_t)rows * sizeof(float) : 0;
}

extern "C" int ofq_fused_layer_norm_min_max_observer(void* stream, const void* x,
                                                     const void* gamma, const void* beta, void* y,
                                                     float* scale, float* zero_point, int t_dtype,
                                                     int64_t rows, int64_t cols, double epsilon,
                                                     int quantization_bit, void* workspace,
                                                     size_t workspace_bytes) {
  return ofq::run(stream, x, nullptr, nullptr, 0.0, false, gamma, beta, y, scale, zero_point,
                  t_dtype, rows, cols, epsilon, quantization_bit, OFQ_LN_STATS_FP32, workspace,
                  workspace_bytes);
}

extern "C" int ofq_fused_skip_layer_norm_min_max_observer(
    void* stream, const void* x, const void* bias, const void* skip, double alpha,
    const void* gamma, const void* beta, void* y, float* scale, float* zero_point, int t_dtype,
    int64_t rows, int64_t cols, double epsilon, int quantization_bit, void* workspace,
    size_t workspace_bytes) {
  return ofq::run(stream, x, bias, skip, alpha, true, gamma, beta, y, scale, zero_point, t_dtype,
                  rows, cols, epsilon, quantization_bit, OFQ_LN_STATS_FP32, workspace,
                  workspace_bytes);
}

extern "C" size_t ofq_fused_layer_norm_quantization_workspace_bytes(int, int64_t rows, int64_t) {
  // [partial maxima: rows floats, padded to 16 bytes][(mean, inv) of every row]
  return rows > 0 ? (((size_t)rows * sizeof(float) + 15) & ~(size_t)15) + (size_t)rows * 2 * sizeof(float)
                  : 0;
}

extern "C" int ofq_fused_layer_norm_quantization(void* stream, const void* x, const void* gamma,
                                                 const void* beta, void* codes, float* scale,
                                                 float* zero_point, int t_dtype, int64_t rows,
                                                 int64_t cols, double epsilon, int quantization_bit,
                                                 int statistics, void* workspace,
                                                 size_t workspace_bytes) {
  using namespace ofq;
  OFQ_RETURN_IF(quantization_bit <= 1 || quantization_bit > 8, OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(statistics != OFQ_LN_STATS_FP32 && statistics != OFQ_LN_STATS_FP64,
                OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(t_dtype != OFQ_F16 && t_dtype != OFQ_BF16 && t_dtype != OFQ_F32,
                OFQ_ERR_BAD_DTYPE);
  OFQ_RETURN_IF(rows < 1 || cols < 1 || rows > 0x7FFFFFFF, OFQ_ERR_BAD_SHAPE);
  OFQ_RETURN_IF(x == nullptr || codes == nullptr || scale == nullptr || zero_point == nullptr,
                OFQ_ERR_NULL_POINTER);
  OFQ_RETURN_IF(workspace == nullptr
                    || workspace_bytes
                           < ofq_fused_layer_norm_quantization_workspace_bytes(t_dtype, rows, cols)
                    || !ofq_aligned16(workspace),
                OFQ_ERR_WORKSPACE);
  // the shapes the register-resident row kernels take; everything else is the two ops in a row
  const int np = (int)(cols / 512);
  if (t_dtype != OFQ_F16 || gamma == nullptr || beta == nullptr || cols % 512 != 0
      || !(np == 1 || np == 2 || np == 4 || np == 8) || !ofq_aligned16(x) || !ofq_aligned16(gamma)
      || !ofq_aligned16(beta) || (reinterpret_cast<uintptr_t>(codes) & 7u) != 0) {
    return OFQ_ERR_UNSUPPORTED;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  float* part = static_cast<float*>(workspace);
  float* stats = reinterpret_cast<float*>(static_cast<uint8_t*>(workspace)
                                          + (((size_t)rows * sizeof(float) + 15) & ~(size_t)15));
  const uint16_t* xs = static_cast<const uint16_t*>(x);
  const uint16_t* gs = static_cast<const uint16_t*>(gamma);
  const uint16_t* bs = static_cast<const uint16_t*>(beta);
  // one row per wave up to 16 waves per CU, beyond that the waves walk the rows; both kernels
  // use the same grid, so a row meets the same wave of the same block twice
  const int64_t waves = rows < 256 * 16 ? rows : 256 * 16;
  constexpr int kWavesPerBlock = kLnqBlock / kWave;
  const int grid = (int)((waves + kWavesPerBlock - 1) / kWavesPerBlock);
  const int64_t nparts = grid;  // one partial maximum per block of the first kernel (<= 512)
  const bool exact = statistics == OFQ_LN_STATS_FP64;
  // parts of a row in the second kernel: enough waves for 16 per CU where the rows allow it
  int split = 1;
  while (split < 4 && split * 2 <= np && waves * split * 2 <= 256 * 16) split *= 2;
  const int grid2 = (grid + 7) / 8 * 8 * split;
#define OFQ_LNQ1(NPV)                                                                           \
  if (exact) {                                                                                  \
    ln_quant_first<NPV, true><<<grid, kLnqBlock, 0, st>>>(xs, gs, bs, part, stats, rows, epsilon);  \
  } else {                                                                                      \
    ln_quant_first<NPV, false><<<grid, kLnqBlock, 0, st>>>(xs, gs, bs, part, stats, rows, epsilon); \
  }
#define OFQ_LNQ2(NPV, SPV)                                                                      \
  if (split == SPV) {                                                                           \
    ln_quant_second<NPV, SPV><<<grid2, kLnqBlock, 0, st>>>(                                     \
        xs, gs, bs, part, nparts, stats, static_cast<int8_t*>(codes), scale, zero_point, rows,  \
        quantization_bit, grid);                                                                \
  }
  switch (np) {
    case 1: OFQ_LNQ1(1) OFQ_LNQ2(1, 1) break;
    case 2: OFQ_LNQ1(2) OFQ_LNQ2(2, 1) OFQ_LNQ2(2, 2) break;
    case 4: OFQ_LNQ1(4) OFQ_LNQ2(4, 1) OFQ_LNQ2(4, 2) OFQ_LNQ2(4, 4) break;
    default: OFQ_LNQ1(8) OFQ_LNQ2(8, 1) OFQ_LNQ2(8, 2) OFQ_LNQ2(8, 4) break;
  }
#undef OFQ_LNQ1
#undef OFQ_LNQ2
  return ofq_check_launch();
}

extern "C" int ofq_fused_layer_norm_min_max_observer_stats(
    void* stream, const void* x, const void* bias, const void* skip, double alpha, int with_skip,
    const void* gamma, const void* beta, void* y, float* scale, float* zero_point, int t_dtype,
    int64_t rows, int64_t cols, double epsilon, int quantization_bit, int statistics,
    void* workspace, size_t workspace_bytes) {
  return ofq::run(stream, x, with_skip ? bias : nullptr, with_skip ? skip : nullptr,
                  with_skip ? alpha : 0.0, with_skip != 0, gamma, beta, y, scale, zero_point,
                  t_dtype, rows, cols, epsilon, quantization_bit, statistics, workspace,
                  workspace_bytes);
}
