// Weight quantiser + packer for gfx950: T[n,k] -> groupwise int4/int8 codes (two 4-bit codes per
// byte, element 2i in the high nibble), scales and zeros in T -- the producer of the format that
// groupwise_dequantize and fused_linear_with_groupwise_quantized_weight consume.  The reference
// defines this format only through the helpers of its own test,
// python/oneflow/test/modules/test_groupwise_quantization.py:26-81, whose arithmetic is followed
// exactly (fp32 throughout, one IEEE division per scale and per element, round half to even,
// codes computed with the unrounded fp32 scale, scale/zero rounded to T at the end):
//   symmetric : scale = absmax / (2^(b-1)-1);  q = rint(x / scale + offset),
//               offset = 2^(b-1)-1 for a uint8 container, 0 for int8
//   asymmetric: scale = (max - min) / (2^b - 1); q = rint((x - min) / scale); zero = min
// A group whose scale is 0 would be 0/0 in that helper; its codes are defined here as `offset`
// (symmetric) or 0 (asymmetric).
//
// Groups along K (the layout every Llama-style checkpoint uses): g/8 lanes share a group, each
// lane owns 8 consecutive elements (one 128-bit load of fp16/bf16), min/max/absmax are folded with
// cross-lane shuffles inside the sub-group, and the lane writes its 8 codes as one 8-byte (int8)
// or 4-byte (int4) store.  Any other grouping takes the strided one-thread-per-group kernel.
#include "ofq_device.h"

namespace ofq {
namespace {

// HALF: v is the value of an fp16 element and `recip` = 1 / sc (IEEE division, once per group):
// the symmetric quotient v / sc is then the twice-corrected product of div_of_half_value, bit for
// bit the division (sc = absmax / 7 or / 127 of fp16 values lies far inside its range).  With 11
// instructions per division this kernel was bound by its arithmetic, not by HBM.
template<bool SYM, bool SIGNED, int BITS, bool HALF = false>
__device__ __forceinline__ int quant_code(float v, float sc, float mn, float recip = 0.f) {
  constexpr float kSignedMax = (float)((1 << (BITS - 1)) - 1);
  constexpr float kOffset = SYM ? (SIGNED ? 0.0f : kSignedMax) : 0.0f;
  float r;
  if (sc == 0.0f) {
    r = kOffset;
  } else if (SYM) {
    const float d = HALF ? div_of_half_value(v, sc, recip) : v / sc;
    r = __builtin_rintf(d + kOffset);
  } else {
    const float d = v - mn;
    r = __builtin_rintf(d / sc);
  }
  return (int)r;
}

template<bool SYM, int BITS>
__device__ __forceinline__ float group_scale(float mn, float mx, float amax) {
  constexpr float kSignedMax = (float)((1 << (BITS - 1)) - 1);
  constexpr float kUnsignedMax = (float)((1 << BITS) - 1);
  return SYM ? amax / kSignedMax : (mx - mn) / kUnsignedMax;
}

// groups along K, g = 8 * L with L a power of two <= 64, rows 16-byte aligned
template<typename T, bool SYM, bool SIGNED, int BITS>
__global__ void __launch_bounds__(256)
quantize_pack_rows(const typename TT<T>::storage* __restrict__ x, uint8_t* __restrict__ q,
                   typename TT<T>::storage* __restrict__ scale,
                   typename TT<T>::storage* __restrict__ zero, int64_t total_groups, int L) {
  typedef typename TT<T>::storage S;
  const int64_t slot = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int lshift = __builtin_ctz((unsigned)L);  // L is a power of two
  const int64_t grp = slot >> lshift;
  const int l = (int)(slot & (L - 1));
  const bool live = grp < total_groups;
  const int64_t base = (live ? grp : 0) * (int64_t)L * 8 + (int64_t)l * 8;
  S raw[8];
  if (sizeof(S) == 2) {
    *reinterpret_cast<u32x4*>(raw) = *reinterpret_cast<const u32x4*>(x + base);
  } else {
    reinterpret_cast<u32x4*>(raw)[0] = reinterpret_cast<const u32x4*>(x + base)[0];
    reinterpret_cast<u32x4*>(raw)[1] = reinterpret_cast<const u32x4*>(x + base)[1];
  }
  float v[8];
  float mn, mx, amax;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    v[e] = TT<T>::load(&raw[e]);
    mn = e == 0 ? v[e] : fminf(mn, v[e]);
    mx = e == 0 ? v[e] : fmaxf(mx, v[e]);
  }
  for (int off = 1; off < L; off <<= 1) {
    mn = fminf(mn, __shfl_xor(mn, off, kWave));
    mx = fmaxf(mx, __shfl_xor(mx, off, kWave));
  }
  amax = fmaxf(fabsf(mn), fabsf(mx));
  const float sc = group_scale<SYM, BITS>(mn, mx, amax);
  if (!live) return;
  if (l == 0) {
    TT<T>::store(&scale[grp], sc);
    if (!SYM) TT<T>::store(&zero[grp], mn);
  }
  uint32_t c[8];
  constexpr bool kHalf = SYM && TT<T>::dtype == OFQ_F16;
  // (an infinite element makes the scale infinite: that group keeps the division)
  const bool fast = kHalf && sc > 0.0f && sc <= 0x1p60f;
  if (fast) {
    const float recip = 1.0f / sc;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      c[e] = (uint32_t)quant_code<SYM, SIGNED, BITS, true>(v[e], sc, mn, recip);
    }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) c[e] = (uint32_t)quant_code<SYM, SIGNED, BITS>(v[e], sc, mn);
  }
  if (BITS == 8) {
    u32x2 w;
    w[0] = (c[0] & 0xFF) | ((c[1] & 0xFF) << 8) | ((c[2] & 0xFF) << 16) | (c[3] << 24);
    w[1] = (c[4] & 0xFF) | ((c[5] & 0xFF) << 8) | ((c[6] & 0xFF) << 16) | (c[7] << 24);
    *reinterpret_cast<u32x2*>(q + base) = w;
  } else {
    uint32_t w = 0;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      w |= ((((c[2 * b] & 0xF) << 4) | (c[2 * b + 1] & 0xF)) << (8 * b));
    }
    *reinterpret_cast<uint32_t*>(q + (base >> 1)) = w;
  }
}

// groups along K of any length that is a multiple of 8 (a whole row per group = per-channel
// quantisation, or lengths the sub-group kernel above does not take): a block per group, 64 to
// 256 threads, two sweeps over the group -- extremes, then codes; the second sweep finds the
// group in cache.  Same arithmetic per element, and max / min do not depend on the order.
template<typename T, bool SYM, bool SIGNED, int BITS>
__global__ void __launch_bounds__(256)
quantize_pack_long_rows(const typename TT<T>::storage* __restrict__ x, uint8_t* __restrict__ q,
                        typename TT<T>::storage* __restrict__ scale,
                        typename TT<T>::storage* __restrict__ zero, int64_t g) {
  typedef typename TT<T>::storage S;
  __shared__ float smem[256 / kWave];
  const int64_t grp = blockIdx.x;
  const S* xg = x + grp * g;
  const int64_t pieces = g >> 3;
  auto load8 = [&](int64_t p, float (&v)[8]) {
    S raw[8];
    if (sizeof(S) == 2) {
      *reinterpret_cast<u32x4*>(raw) = *reinterpret_cast<const u32x4*>(xg + p * 8);
    } else {
      reinterpret_cast<u32x4*>(raw)[0] = reinterpret_cast<const u32x4*>(xg + p * 8)[0];
      reinterpret_cast<u32x4*>(raw)[1] = reinterpret_cast<const u32x4*>(xg + p * 8)[1];
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = TT<T>::load(&raw[e]);
  };
  float mn = __builtin_inff(), mx = -__builtin_inff();
  for (int64_t p = threadIdx.x; p < pieces; p += blockDim.x) {
    float v[8];
    load8(p, v);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      mn = fminf(mn, v[e]);
      mx = fmaxf(mx, v[e]);
    }
  }
  mn = block_reduce(mn, OpMin(), smem);
  mx = block_reduce(mx, OpMax(), smem);
  const float amax = fmaxf(fabsf(mn), fabsf(mx));
  const float sc = group_scale<SYM, BITS>(mn, mx, amax);
  if (threadIdx.x == 0) {
    TT<T>::store(&scale[grp], sc);
    if (!SYM) TT<T>::store(&zero[grp], mn);
  }
  const int64_t base = grp * g;
  for (int64_t p = threadIdx.x; p < pieces; p += blockDim.x) {
    float v[8];
    load8(p, v);
    uint32_t c[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) c[e] = (uint32_t)quant_code<SYM, SIGNED, BITS>(v[e], sc, mn);
    if (BITS == 8) {
      u32x2 w;
      w[0] = (c[0] & 0xFF) | ((c[1] & 0xFF) << 8) | ((c[2] & 0xFF) << 16) | (c[3] << 24);
      w[1] = (c[4] & 0xFF) | ((c[5] & 0xFF) << 8) | ((c[6] & 0xFF) << 16) | (c[7] << 24);
      *reinterpret_cast<u32x2*>(q + base + p * 8) = w;
    } else {
      uint32_t w = 0;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        w |= ((((c[2 * b] & 0xF) << 4) | (c[2 * b + 1] & 0xF)) << (8 * b));
      }
      *reinterpret_cast<uint32_t*>(q + ((base + p * 8) >> 1)) = w;
    }
  }
}

// any grouping: x viewed as [outer][groups][g][inner]; one thread per (outer, group, column) for
// 8-bit codes, per (outer, group, column pair) for 4-bit codes packed along the inner axis, per
// (outer, group) when inner == 1 (pairs then lie inside the group, g is even)
template<typename T, bool SYM, bool SIGNED, int BITS>
__global__ void __launch_bounds__(256)
quantize_pack_generic(const typename TT<T>::storage* __restrict__ x, uint8_t* __restrict__ q,
                      typename TT<T>::storage* __restrict__ scale,
                      typename TT<T>::storage* __restrict__ zero, int64_t og, int64_t g,
                      int64_t inner) {
  // cols: number of independent columns a thread handles (2 when packing pairs across columns)
  const bool pair_cols = BITS == 4 && inner > 1;
  const int64_t cols_per_thread = pair_cols ? 2 : 1;
  const int64_t threads_per_og = inner / cols_per_thread;
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= og * threads_per_og) return;
  const int64_t o = t / threads_per_og;
  const int64_t i0 = (t - o * threads_per_og) * cols_per_thread;
  float sc[2], mn[2];
  for (int64_t cI = 0; cI < cols_per_thread; ++cI) {
    const int64_t i = i0 + cI;
    float lo = 0.f, hi = 0.f;
    for (int64_t j = 0; j < g; ++j) {
      const float v = TT<T>::load(&x[(o * g + j) * inner + i]);
      lo = j == 0 ? v : fminf(lo, v);
      hi = j == 0 ? v : fmaxf(hi, v);
    }
    const float amax = fmaxf(fabsf(lo), fabsf(hi));
    sc[cI] = group_scale<SYM, BITS>(lo, hi, amax);
    mn[cI] = lo;
    TT<T>::store(&scale[o * inner + i], sc[cI]);
    if (!SYM) TT<T>::store(&zero[o * inner + i], lo);
  }
  if (BITS == 8) {
    for (int64_t j = 0; j < g; ++j) {
      const int64_t idx = (o * g + j) * inner + i0;
      q[idx] = (uint8_t)quant_code<SYM, SIGNED, BITS>(TT<T>::load(&x[idx]), sc[0], mn[0]);
    }
  } else if (pair_cols) {
    for (int64_t j = 0; j < g; ++j) {
      const int64_t idx = (o * g + j) * inner + i0;  // even: i0 is even and inner is even
      const int a = quant_code<SYM, SIGNED, BITS>(TT<T>::load(&x[idx]), sc[0], mn[0]);
      const int b = quant_code<SYM, SIGNED, BITS>(TT<T>::load(&x[idx + 1]), sc[1], mn[1]);
      q[idx >> 1] = (uint8_t)(((a & 0xF) << 4) | (b & 0xF));
    }
  } else {
    for (int64_t j = 0; j < g; j += 2) {
      const int64_t idx = (o * g + j) * inner + i0;  // inner == 1, g even: idx is even
      const int a = quant_code<SYM, SIGNED, BITS>(TT<T>::load(&x[idx]), sc[0], mn[0]);
      const int b = quant_code<SYM, SIGNED, BITS>(TT<T>::load(&x[idx + 1]), sc[0], mn[0]);
      q[idx >> 1] = (uint8_t)(((a & 0xF) << 4) | (b & 0xF));
    }
  }
}

template<typename T, bool SYM, bool SIGNED, int BITS>
int launch_variant(hipStream_t st, const void* x, void* q, void* scale, void* zero, int group_dim,
                   int64_t g, int64_t n, int64_t k) {
  typedef typename TT<T>::storage S;
  const S* xs = static_cast<const S*>(x);
  uint8_t* qs = static_cast<uint8_t*>(q);
  S* ss = static_cast<S*>(scale);
  S* zs = static_cast<S*>(zero);
  const int64_t outer = group_dim == 0 ? 1 : n;
  const int64_t groups = (group_dim == 0 ? n : k) / g;
  const int64_t inner = group_dim == 0 ? k : 1;
  const int64_t og = outer * groups;
  const int64_t L = g / 8;
  const bool fast = group_dim == 1 && g % 8 == 0 && L <= 64 && (L & (L - 1)) == 0
                    && ofq_aligned16(x) && ((reinterpret_cast<uintptr_t>(q) & 7u) == 0);
  if (fast) {
    const int64_t slots = og * L;
    const int64_t grid = (slots + 255) / 256;
    if (grid > 0x7FFFFFFF) return OFQ_ERR_UNSUPPORTED;
    quantize_pack_rows<T, SYM, SIGNED, BITS><<<(int)grid, 256, 0, st>>>(xs, qs, ss, zs, og, (int)L);
  } else if (group_dim == 1 && g % 8 == 0 && ofq_aligned16(x)
             && ((reinterpret_cast<uintptr_t>(q) & 7u) == 0) && og <= 0x7FFFFFFF) {
    int threads = (int)((L + 63) / 64 * 64);
    if (threads > 256) threads = 256;
    quantize_pack_long_rows<T, SYM, SIGNED, BITS><<<(int)og, threads, 0, st>>>(xs, qs, ss, zs, g);
  } else {
    const int64_t threads = og * (inner / ((BITS == 4 && inner > 1) ? 2 : 1));
    const int64_t grid = (threads + 255) / 256;
    if (grid > 0x7FFFFFFF) return OFQ_ERR_UNSUPPORTED;
    quantize_pack_generic<T, SYM, SIGNED, BITS><<<(int)grid, 256, 0, st>>>(xs, qs, ss, zs, og, g,
                                                                         inner);
  }
  return ofq_check_launch();
}

template<typename T>
int launch_t(hipStream_t st, const void* x, void* q, void* scale, void* zero, bool is_signed,
             int bits, bool symmetric, int group_dim, int64_t g, int64_t n, int64_t k) {
#define OFQ_QV(SYMV, SGV, BV)                                          \
  if (symmetric == SYMV && is_signed == SGV && bits == BV)             \
    return launch_variant<T, SYMV, SGV, BV>(st, x, q, scale, zero, group_dim, g, n, k);
  OFQ_QV(true, true, 4)
  OFQ_QV(true, false, 4)
  OFQ_QV(false, false, 4)
  OFQ_QV(true, true, 8)
  OFQ_QV(true, false, 8)
  OFQ_QV(false, false, 8)
#undef OFQ_QV
  return OFQ_ERR_UNSUPPORTED;
}

}  // namespace
}  // namespace ofq

extern "C" int ofq_groupwise_quantize(void* stream, const void* x, void* q, void* scale,
                                      void* zero, int t_dtype, int q_dtype, int num_bits,
                                      int symmetric, int group_dim, int64_t group_size, int64_t n,
                                      int64_t k) {
  OFQ_RETURN_IF(num_bits != 4 && num_bits != 8, OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(group_dim != 0 && group_dim != 1, OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(q_dtype != OFQ_U8 && q_dtype != OFQ_I8, OFQ_ERR_BAD_DTYPE);
  OFQ_RETURN_IF(!symmetric && q_dtype != OFQ_U8, OFQ_ERR_BAD_DTYPE);
  OFQ_RETURN_IF(t_dtype != OFQ_F16 && t_dtype != OFQ_BF16 && t_dtype != OFQ_F32,
                OFQ_ERR_BAD_DTYPE);
  OFQ_RETURN_IF(n < 0 || k < 0 || group_size <= 0, OFQ_ERR_BAD_SHAPE);
  if (n == 0 || k == 0) return OFQ_OK;
  const int64_t dim = group_dim == 0 ? n : k;
  OFQ_RETURN_IF(group_size > dim || dim % group_size != 0, OFQ_ERR_BAD_SHAPE);
  // two codes per byte along k; with groups along k a pair must not straddle two groups
  OFQ_RETURN_IF(num_bits == 4 && (k % 2 != 0 || (group_dim == 1 && group_size % 2 != 0)),
                OFQ_ERR_BAD_SHAPE);
  OFQ_RETURN_IF(x == nullptr || q == nullptr || scale == nullptr, OFQ_ERR_NULL_POINTER);
  OFQ_RETURN_IF((symmetric != 0) != (zero == nullptr), OFQ_ERR_NULL_POINTER);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool sg = q_dtype == OFQ_I8;
  const bool sym = symmetric != 0;
  switch (t_dtype) {
    case OFQ_F16:
      return ofq::launch_t<ofq::f16>(st, x, q, scale, zero, sg, num_bits, sym, group_dim,
                                     group_size, n, k);
    case OFQ_BF16:
      return ofq::launch_t<ofq::bf16>(st, x, q, scale, zero, sg, num_bits, sym, group_dim,
                                      group_size, n, k);
    default:
      return ofq::launch_t<float>(st, x, q, scale, zero, sg, num_bits, sym, group_dim, group_size,
                                  n, k);
  }
}
