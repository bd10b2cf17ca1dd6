// Register-level dequantisation shared by the GEMM weight feeder and the decode kernels:
// packed integer codes in, values of T in NATURAL element order out, formed exactly as the
// reference does, w~ = T(T(q) * s) + z with one rounding per operation
// (oneflow/user/kernels/groupwise_quantization_kernels.cu:73-117).
#pragma once

#include "ofq_device.h"

namespace ofq {
namespace {

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

// two floats -> packed bf16 pair (round to nearest even), first in the low half
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  const f32x2 p = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(p, bf16x2_t));
}

// bf16 pair `r` plus z in fp32, rounded to bf16 again
__device__ __forceinline__ uint32_t add_bf16_pair(uint32_t r, float z) {
  return pack_bf16(__builtin_bit_cast(float, r << 16) + z,
                   __builtin_bit_cast(float, r & 0xFFFF0000u) + z);
}

// 16 values of T (two 128-bit pieces) from 16 byte codes.
// bf16: v_cvt_f32_ubyteN, v_mul_f32 (v_fma_f32 for a signed container: the codes are read as
// offset binary and the offset is taken out inside the fused multiply-add, which is exact),
// v_cvt_pk_bf16_f32, and for a zero term re-widen, v_add_f32, v_cvt_pk_bf16_f32.
// fp16: the 0x6400 trick with packed fp16 math (2 instructions per element).
template<typename T, bool SIGNED, int ZMODE>
__device__ __forceinline__ void dequant16_b8(const u32x4 codes, float s, float z, u32x4& o0,
                                             u32x4& o1) {
  uint32_t r[8];
  if constexpr (TT<T>::dtype == OFQ_BF16) {
    const float off = SIGNED ? -128.0f * s : 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      uint32_t x = codes[w];
      if (SIGNED) x ^= 0x80808080u;
      float p[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float u = (float)((x >> (8 * e)) & 0xFFu);
        p[e] = SIGNED ? __builtin_fmaf(u, s, off) : u * s;
      }
      uint32_t r01 = pack_bf16(p[0], p[1]);
      uint32_t r23 = pack_bf16(p[2], p[3]);
      if (ZMODE != 0) {
        r01 = add_bf16_pair(r01, z);
        r23 = add_bf16_pair(r23, z);
      }
      r[2 * w] = r01;
      r[2 * w + 1] = r23;
    }
  } else if constexpr (TT<T>::dtype == OFQ_F16) {
    const f16 sh = (f16)s, zh = (f16)z;  // s and z were widened from fp16: exact
    const f16x2 s2 = {sh, sh}, z2 = {zh, zh};
    const f16 off = SIGNED ? (f16)(-1152.0f) : (f16)(-1024.0f);
    const f16x2 off2 = {off, off};
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      uint32_t word = codes[w];
      if (SIGNED) word ^= 0x80808080u;
      f16x2 a = __builtin_bit_cast(f16x2, __builtin_amdgcn_perm(word, 0x64646464u, 0x00050004u)) + off2;
      f16x2 b = __builtin_bit_cast(f16x2, __builtin_amdgcn_perm(word, 0x64646464u, 0x00070006u)) + off2;
      a = a * s2;
      b = b * s2;
      if (ZMODE != 0) {
        a = a + z2;
        b = b + z2;
      }
      r[2 * w] = __builtin_bit_cast(uint32_t, a);
      r[2 * w + 1] = __builtin_bit_cast(uint32_t, b);
    }
  } else {
    typename TT<T>::storage vals[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const uint32_t b = (codes[e >> 2] >> ((e & 3) * 8)) & 0xFFu;
      const int code = SIGNED ? (int)(int8_t)b : (int)b;
      float v = TT<T>::round((float)code * s);
      if (ZMODE != 0) v = v + z;
      TT<T>::store(&vals[e], v);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = reinterpret_cast<const uint32_t*>(vals)[i];
  }
  o0 = u32x4{r[0], r[1], r[2], r[3]};
  o1 = u32x4{r[4], r[5], r[6], r[7]};
}

// 8 values of T (fp16 or bf16, one 128-bit piece) from one word of 4-bit codes.  Element 2b is
// the high nibble of byte b, element 2b+1 its low nibble
// (groupwise_quantization_kernels.cu:44-57).
template<typename T, bool SIGNED, int ZMODE>
__device__ __forceinline__ u32x4 dequant8_b4(uint32_t word, float s, float z) {
  static_assert(TT<T>::dtype == OFQ_BF16 || TT<T>::dtype == OFQ_F16, "16-bit T only");
  if (SIGNED) word ^= 0x88888888u;  // two's complement nibbles -> offset binary
  const uint32_t hi = (word >> 4) & 0x0F0F0F0Fu;  // elements 0, 2, 4, 6
  const uint32_t lo = word & 0x0F0F0F0Fu;         // elements 1, 3, 5, 7
  u32x4 o;
  if constexpr (TT<T>::dtype == OFQ_BF16) {
    const float off = SIGNED ? -8.0f * s : 0.f;
    // the two masked words stay as they are, so that byte b of each converts with one
    // v_cvt_f32_ubyte<b>; folded into the original word every element costs a bit-field
    // extract in front of its conversion
    uint32_t hi_pinned = hi, lo_pinned = lo;
    asm("" : "+v"(hi_pinned));
    asm("" : "+v"(lo_pinned));
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const float u0 = (float)((hi_pinned >> (8 * b)) & 0xFFu);
      const float u1 = (float)((lo_pinned >> (8 * b)) & 0xFFu);
      const float p0 = SIGNED ? __builtin_fmaf(u0, s, off) : u0 * s;
      const float p1 = SIGNED ? __builtin_fmaf(u1, s, off) : u1 * s;
      uint32_t r = pack_bf16(p0, p1);
      if (ZMODE != 0) r = add_bf16_pair(r, z);
      o[b] = r;
    }
  } else {
    const f16 sh = (f16)s, zh = (f16)z;
    const f16x2 s2 = {sh, sh}, z2 = {zh, zh};
    const f16 off = SIGNED ? (f16)(-1032.0f) : (f16)(-1024.0f);
    const f16x2 off2 = {off, off};
    const uint32_t sel[4] = {0x0C000C04u, 0x0C010C05u, 0x0C020C06u, 0x0C030C07u};
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      // (hi.byte b, 0, lo.byte b, 0) | 0x64006400 = the half pair (1024 + e_2b, 1024 + e_2b+1)
      const uint32_t pr = __builtin_amdgcn_perm(hi, lo, sel[b]) | 0x64006400u;
      f16x2 v = (__builtin_bit_cast(f16x2, pr) + off2) * s2;
      if (ZMODE != 0) v = v + z2;
      o[b] = __builtin_bit_cast(uint32_t, v);
    }
  }
  return o;
}

// ---- one scale (and zero) PER ELEMENT: groups that run along N, so that the scale of an element
// depends on its k (scale / zero of shape [N / group_size, K]).  `s` / `z` hold the T values of
// the same 8 consecutive k as the codes, two per word, as they lie in memory. ----

// bf16 pair `r` plus bf16 pair `zw`, element-wise in fp32, rounded to bf16 again
__device__ __forceinline__ uint32_t add_bf16_pairs(uint32_t r, uint32_t zw) {
  return pack_bf16(__builtin_bit_cast(float, r << 16) + __builtin_bit_cast(float, zw << 16),
                   __builtin_bit_cast(float, r & 0xFFFF0000u)
                       + __builtin_bit_cast(float, zw & 0xFFFF0000u));
}

// the zero term of a symmetric quantisation in an unsigned container, T(-(2^(b-1)-1) * s), for a
// pair of scales
template<typename T, int BITS>
__device__ __forceinline__ uint32_t sym_zero_pair(uint32_t sw) {
  constexpr float kNeg = -(float)((1 << (BITS - 1)) - 1);
  if constexpr (TT<T>::dtype == OFQ_BF16) {
    return pack_bf16(kNeg * __builtin_bit_cast(float, sw << 16),
                     kNeg * __builtin_bit_cast(float, sw & 0xFFFF0000u));
  } else {
    const f16x2 c = {(f16)kNeg, (f16)kNeg};
    return __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, sw) * c);
  }
}

// (u0, u1): two codes as offset-binary integers 0 .. 2^BITS - 1 in fp32 -> pair of w~ in T
template<typename T, int BITS, bool SIGNED, int ZMODE>
__device__ __forceinline__ uint32_t dequant_pair_bf16(float u0, float u1, uint32_t sw, uint32_t zw) {
  const float s0 = __builtin_bit_cast(float, sw << 16);
  const float s1 = __builtin_bit_cast(float, sw & 0xFFFF0000u);
  constexpr float kOff = -(float)(1 << (BITS - 1));
  // a signed container is read as offset binary; (u - 2^(b-1)) * s is exact inside the fma
  const float p0 = SIGNED ? __builtin_fmaf(u0, s0, kOff * s0) : u0 * s0;
  const float p1 = SIGNED ? __builtin_fmaf(u1, s1, kOff * s1) : u1 * s1;
  uint32_t r = pack_bf16(p0, p1);
  if (ZMODE == 2) r = add_bf16_pairs(r, zw);
  if (ZMODE == 1) r = add_bf16_pairs(r, sym_zero_pair<T, BITS>(sw));
  return r;
}

template<typename T, bool SIGNED, int ZMODE>
__device__ __forceinline__ u32x4 dequant8_b4_v(uint32_t word, const u32x4 s, const u32x4 z) {
  static_assert(TT<T>::dtype == OFQ_BF16 || TT<T>::dtype == OFQ_F16, "16-bit T only");
  if (SIGNED) word ^= 0x88888888u;
  const uint32_t hi = (word >> 4) & 0x0F0F0F0Fu;  // elements 0, 2, 4, 6
  const uint32_t lo = word & 0x0F0F0F0Fu;         // elements 1, 3, 5, 7
  u32x4 o;
  if constexpr (TT<T>::dtype == OFQ_BF16) {
    uint32_t hi_pinned = hi, lo_pinned = lo;  // as in dequant8_b4
    asm("" : "+v"(hi_pinned));
    asm("" : "+v"(lo_pinned));
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const float u0 = (float)((hi_pinned >> (8 * b)) & 0xFFu);
      const float u1 = (float)((lo_pinned >> (8 * b)) & 0xFFu);
      o[b] = dequant_pair_bf16<T, 4, SIGNED, ZMODE>(u0, u1, s[b], z[b]);
    }
  } else {
    const f16 off = SIGNED ? (f16)(-1032.0f) : (f16)(-1024.0f);
    const f16x2 off2 = {off, off};
    const uint32_t sel[4] = {0x0C000C04u, 0x0C010C05u, 0x0C020C06u, 0x0C030C07u};
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const uint32_t pr = __builtin_amdgcn_perm(hi, lo, sel[b]) | 0x64006400u;
      // the words go through scalars of their own: a bit cast applied directly to s[b] was
      // seen to read element 0 for every b
      const uint32_t sw = s[b];
      const uint32_t zw = z[b];
      f16x2 v = (__builtin_bit_cast(f16x2, pr) + off2) * __builtin_bit_cast(f16x2, sw);
      if (ZMODE == 2) v = v + __builtin_bit_cast(f16x2, zw);
      if (ZMODE == 1) v = v + __builtin_bit_cast(f16x2, sym_zero_pair<T, 4>(sw));
      o[b] = __builtin_bit_cast(uint32_t, v);
    }
  }
  return o;
}

// 16 byte codes with 16 scales: s0 / z0 belong to elements 0..7, s1 / z1 to elements 8..15
template<typename T, bool SIGNED, int ZMODE>
__device__ __forceinline__ void dequant16_b8_v(const u32x4 codes, const u32x4 s0, const u32x4 s1,
                                               const u32x4 z0, const u32x4 z1, u32x4& o0,
                                               u32x4& o1) {
  static_assert(TT<T>::dtype == OFQ_BF16 || TT<T>::dtype == OFQ_F16, "16-bit T only");
  uint32_t r[8];
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    uint32_t word = codes[w];
    if (SIGNED) word ^= 0x80808080u;
    // elements 4w .. 4w+3: scale words 2w and 2w+1 of the sixteen
    const uint32_t sa = w < 2 ? s0[2 * w] : s1[2 * w - 4];
    const uint32_t sb = w < 2 ? s0[2 * w + 1] : s1[2 * w - 3];
    const uint32_t za = w < 2 ? z0[2 * w] : z1[2 * w - 4];
    const uint32_t zb = w < 2 ? z0[2 * w + 1] : z1[2 * w - 3];
    if constexpr (TT<T>::dtype == OFQ_BF16) {
      float u[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) u[e] = (float)((word >> (8 * e)) & 0xFFu);
      r[2 * w] = dequant_pair_bf16<T, 8, SIGNED, ZMODE>(u[0], u[1], sa, za);
      r[2 * w + 1] = dequant_pair_bf16<T, 8, SIGNED, ZMODE>(u[2], u[3], sb, zb);
    } else {
      const f16 off = SIGNED ? (f16)(-1152.0f) : (f16)(-1024.0f);
      const f16x2 off2 = {off, off};
      f16x2 a = __builtin_bit_cast(f16x2, __builtin_amdgcn_perm(word, 0x64646464u, 0x00050004u)) + off2;
      f16x2 b = __builtin_bit_cast(f16x2, __builtin_amdgcn_perm(word, 0x64646464u, 0x00070006u)) + off2;
      a = a * __builtin_bit_cast(f16x2, sa);
      b = b * __builtin_bit_cast(f16x2, sb);
      if (ZMODE == 2) {
        a = a + __builtin_bit_cast(f16x2, za);
        b = b + __builtin_bit_cast(f16x2, zb);
      }
      if (ZMODE == 1) {
        a = a + __builtin_bit_cast(f16x2, sym_zero_pair<T, 8>(sa));
        b = b + __builtin_bit_cast(f16x2, sym_zero_pair<T, 8>(sb));
      }
      r[2 * w] = __builtin_bit_cast(uint32_t, a);
      r[2 * w + 1] = __builtin_bit_cast(uint32_t, b);
    }
  }
  o0 = u32x4{r[0], r[1], r[2], r[3]};
  o1 = u32x4{r[4], r[5], r[6], r[7]};
}

}  // namespace
}  // namespace ofq
