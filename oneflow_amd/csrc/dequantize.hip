// groupwise_dequantize for gfx950.
//
// Semantics (oneflow/user/kernels/groupwise_quantization_kernels.cu:170-203, :275-299):
//   view out as [outer][group_size][inner]; out = T( T(T(q) * scale[outer][inner]) + zero ),
//   zero = zero[outer][inner] (asymmetric), -T(2^(b-1)-1)*scale (symmetric, uint8 container) or
//   0 (symmetric, int8 container).  Both operations round to T.
//
// The op is pure streaming: 1 (or 1/2) byte in, sizeof(T) bytes out per element, so every
// variant is a grid-stride loop of 128-bit loads and stores; what differs is how many elements a
// lane owns and where its scale comes from.
#include "ofq_device.h"

namespace ofq {
namespace {

template<typename T, int BITS, bool SIGNED, bool SYM>
__device__ __forceinline__ float zero_term(const typename TT<T>::storage* zero, int64_t idx,
                                           float s) {
  if (!SYM) return TT<T>::load(zero + idx);
  if (SIGNED) return 0.0f;
  return TT<T>::round(-(float)((1 << (BITS - 1)) - 1) * s);
}

// ---- any shape, one element per lane ----------------------------------------------------
template<typename T, int BITS, bool SIGNED, bool SYM>
__global__ void __launch_bounds__(256)
dequant_scalar(const uint8_t* __restrict__ q, const typename TT<T>::storage* __restrict__ scale,
               const typename TT<T>::storage* __restrict__ zero,
               typename TT<T>::storage* __restrict__ out, int64_t elem_cnt, int64_t group_size,
               int64_t inner) {
  const int64_t step = (int64_t)gridDim.x * blockDim.x;
  const int64_t gi = group_size * inner;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < elem_cnt; i += step) {
    const int64_t o = i / gi;
    const int64_t in_i = (i - o * gi) % inner;
    const int64_t si = o * inner + in_i;
    const float s = TT<T>::load(scale + si);
    const float z = zero_term<T, BITS, SIGNED, SYM>(zero, si, s);
    const float c = (float)code_at<BITS, SIGNED>(q, i);
    TT<T>::store(out + i, TT<T>::round(c * s) + z);
  }
}

// ---- 8 consecutive elements per lane; scale is a scalar per lane (INNER1) or a vector ------
// INNER1: the group axis is the innermost one and 8 | group_size.
// else  : 8 | inner, the lane's 8 elements share (outer, group row) and use 8 scales.
template<typename T, int BITS, bool SIGNED, bool SYM, bool INNER1>
__global__ void __launch_bounds__(256)
dequant_vec8(const uint8_t* __restrict__ q, const typename TT<T>::storage* __restrict__ scale,
             const typename TT<T>::storage* __restrict__ zero,
             typename TT<T>::storage* __restrict__ out, int64_t n_packs, int64_t group_size,
             int64_t inner) {
  typedef typename TT<T>::storage S;
  const int64_t step = (int64_t)gridDim.x * blockDim.x;
  const int64_t packs_per_group = group_size / 8;             // INNER1
  const int64_t packed_inner = inner / 8;                     // !INNER1
  const int64_t packed_gi = group_size * packed_inner;        // !INNER1
  for (int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; p < n_packs; p += step) {
    uint32_t codes[2];
    if (BITS == 8) {
      const u32x2 v = *reinterpret_cast<const u32x2*>(q + p * 8);
      codes[0] = v.x;
      codes[1] = v.y;
    } else {
      codes[0] = *reinterpret_cast<const uint32_t*>(q + p * 4);
      codes[1] = 0;
    }
    float s[8], z[8];
    if (INNER1) {
      const int64_t g = p / packs_per_group;
      const float sv = TT<T>::load(scale + g);
      const float zv = zero_term<T, BITS, SIGNED, SYM>(zero, g, sv);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        s[e] = sv;
        z[e] = zv;
      }
    } else {
      const int64_t o = p / packed_gi;
      const int64_t in_p = (p - o * packed_gi) % packed_inner;
      const int64_t si = (o * packed_inner + in_p) * 8;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        s[e] = TT<T>::load(scale + si + e);
        z[e] = zero_term<T, BITS, SIGNED, SYM>(zero, si + e, s[e]);
      }
    }
    S r[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      int c;
      if (BITS == 8) {
        const uint32_t b = (codes[e >> 2] >> ((e & 3) * 8)) & 0xFFu;
        c = SIGNED ? (int)(int8_t)b : (int)b;
      } else {
        // byte e/2 of the word; even element = high nibble
        const uint32_t b = (codes[0] >> ((e >> 1) * 8)) & 0xFFu;
        const int nib = (e & 1) ? (b & 0xF) : (b >> 4);
        c = SIGNED ? ((nib ^ 8) - 8) : nib;
      }
      TT<T>::store(&r[e], TT<T>::round((float)c * s[e]) + z[e]);
    }
    S* dst = out + p * 8;
    if (sizeof(S) == 2) {
      *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(r);
    } else {
      *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(r);
      *reinterpret_cast<u32x4*>(dst + 4) = *reinterpret_cast<const u32x4*>(r + 4);
    }
  }
}

// ---- fp16, 8-bit codes, group axis innermost, 8 | group_size: native packed fp16 math ------
// A lane owns two packs of 8 codes, 64 packs apart: each of its two 64-bit loads is one of 64
// consecutive ones (512 contiguous bytes per wave instruction) and each of its two 128-bit stores
// one of 64 consecutive ones (1 KB per instruction) -- a lane that owned 16 consecutive codes
// would write its 32 bytes as two interleaved half-used store instructions (measured 6 % slower).
// Bytes are turned into fp16 by the 0x6400 trick: the half with bits 0x6400|b is exactly
// 1024 + b, so one v_perm_b32 builds two halves and one packed subtract recovers the code.
template<bool SIGNED, bool SYM>
__device__ __forceinline__ u32x4 dequant8_f16_b8(u32x2 c, f16 s, f16 zin) {
  f16 z = zin;
  if (SYM) z = SIGNED ? (f16)0.0f : (f16)(-127.0f) * s;
  const f16x2 s2 = {s, s};
  const f16x2 z2 = {z, z};
  const f16 off = SIGNED ? (f16)(-1152.0f) : (f16)(-1024.0f);
  const f16x2 off2 = {off, off};
  uint32_t r[4];
#pragma unroll
  for (int w = 0; w < 2; ++w) {
    uint32_t word = c[w];
    if (SIGNED) word ^= 0x80808080u;  // two's complement -> offset binary
    const uint32_t lo = __builtin_amdgcn_perm(word, 0x64646464u, 0x00050004u);
    const uint32_t hi = __builtin_amdgcn_perm(word, 0x64646464u, 0x00070006u);
    f16x2 a = __builtin_bit_cast(f16x2, lo) + off2;
    f16x2 b = __builtin_bit_cast(f16x2, hi) + off2;
    a = a * s2;
    b = b * s2;
    if (!(SYM && SIGNED)) {
      a = a + z2;
      b = b + z2;
    }
    r[2 * w] = __builtin_bit_cast(uint32_t, a);
    r[2 * w + 1] = __builtin_bit_cast(uint32_t, b);
  }
  return u32x4{r[0], r[1], r[2], r[3]};
}

template<bool SIGNED, bool SYM, int PPL>
__global__ void __launch_bounds__(256)
dequant_f16_b8_rows(const u32x2* __restrict__ q, const f16* __restrict__ scale,
                    const f16* __restrict__ zero, u32x4* __restrict__ out, int64_t n_packs,
                    int64_t packs_per_group) {
  // wave chunk = 64 * PPL consecutive packs; lane l takes packs l, 64 + l, ... of the chunk
  const int lane = threadIdx.x & 63;
  const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const int64_t nwaves = ((int64_t)gridDim.x * blockDim.x) >> 6;
  for (int64_t base = wave * (64 * PPL); base < n_packs; base += nwaves * (64 * PPL)) {
    u32x2 c[PPL];
    f16 s[PPL], z[PPL];
    bool v[PPL];
#pragma unroll
    for (int i = 0; i < PPL; ++i) {
      const int64_t p = base + i * 64 + lane;
      v[i] = p < n_packs;
      c[i] = u32x2{0u, 0u};
      if (v[i]) c[i] = __builtin_nontemporal_load(q + p);
      const int64_t g = (v[i] ? p : 0) / packs_per_group;
      s[i] = scale[g];
      z[i] = SYM ? (f16)0.0f : zero[g];
    }
#pragma unroll
    for (int i = 0; i < PPL; ++i) {
      const int64_t p = base + i * 64 + lane;
      if (v[i]) __builtin_nontemporal_store(dequant8_f16_b8<SIGNED, SYM>(c[i], s[i], z[i]), out + p);
    }
  }
}

inline int grid_for(int64_t items, int block) {
  int64_t g = (items + block - 1) / block;
  const int64_t cap = 256 * 32;  // 256 CUs x enough resident blocks to cover HBM latency
  if (g > cap) g = cap;
  if (g < 1) g = 1;
  return (int)g;
}

template<typename T, int BITS, bool SIGNED, bool SYM>
int launch(hipStream_t st, const void* in, const void* scale, const void* zero, void* out,
           int64_t outer, int64_t group_size, int64_t inner) {
  typedef typename TT<T>::storage S;
  const int64_t elem_cnt = outer * group_size * inner;
  const uint8_t* q = static_cast<const uint8_t*>(in);
  const S* sc = static_cast<const S*>(scale);
  const S* ze = static_cast<const S*>(zero);
  S* o = static_cast<S*>(out);
  if constexpr (BITS == 8 && sizeof(S) == 2 && TT<T>::dtype == OFQ_F16) {
    if (inner == 1 && group_size % 8 == 0) {
      const int64_t n_packs = elem_cnt / 8;
      // two packs per lane; more packs per lane or more blocks per CU measure the same
      dequant_f16_b8_rows<SIGNED, SYM, 2><<<grid_for((n_packs + 1) / 2, 256), 256, 0, st>>>(
          reinterpret_cast<const u32x2*>(q), sc, ze, reinterpret_cast<u32x4*>(o), n_packs,
          group_size / 8);
      return ofq_check_launch();
    }
  }
  if (inner == 1 && group_size % 8 == 0) {
    const int64_t n_packs = elem_cnt / 8;
    dequant_vec8<T, BITS, SIGNED, SYM, true><<<grid_for(n_packs, 256), 256, 0, st>>>(
        q, sc, ze, o, n_packs, group_size, inner);
  } else if (inner > 1 && inner % 8 == 0) {
    const int64_t n_packs = elem_cnt / 8;
    dequant_vec8<T, BITS, SIGNED, SYM, false><<<grid_for(n_packs, 256), 256, 0, st>>>(
        q, sc, ze, o, n_packs, group_size, inner);
  } else {
    dequant_scalar<T, BITS, SIGNED, SYM><<<grid_for(elem_cnt, 256), 256, 0, st>>>(
        q, sc, ze, o, elem_cnt, group_size, inner);
  }
  return ofq_check_launch();
}

template<typename T>
int dispatch(hipStream_t st, const void* in, const void* scale, const void* zero, void* out,
             bool is_signed, int bits, bool sym, int64_t outer, int64_t group_size,
             int64_t inner) {
#define OFQ_CASE(B, SG, SY)                                                          \
  if (bits == B && is_signed == SG && sym == SY)                                     \
    return launch<T, B, SG, SY>(st, in, scale, zero, out, outer, group_size, inner);
  OFQ_CASE(8, false, true)
  OFQ_CASE(8, true, true)
  OFQ_CASE(8, false, false)
  OFQ_CASE(4, false, true)
  OFQ_CASE(4, true, true)
  OFQ_CASE(4, false, false)
#undef OFQ_CASE
  return OFQ_ERR_UNSUPPORTED;
}

}  // namespace
}  // namespace ofq

extern "C" int ofq_groupwise_dequantize(void* stream, const void* in, const void* scale,
                                        const void* zero, void* out, int in_dtype, int t_dtype,
                                        int num_bits, int symmetric, int64_t outer,
                                        int64_t group_size, int64_t inner) {
  OFQ_RETURN_IF(num_bits != 4 && num_bits != 8, OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(in_dtype != OFQ_U8 && in_dtype != OFQ_I8, OFQ_ERR_BAD_DTYPE);
  // asymmetric codes are unsigned: fused_linear_with_groupwise_quantized_weight_op.cpp:89-90,
  // functional/impl/quantization.cpp:179-182
  OFQ_RETURN_IF(!symmetric && in_dtype != OFQ_U8, OFQ_ERR_BAD_DTYPE);
  OFQ_RETURN_IF(t_dtype != OFQ_F16 && t_dtype != OFQ_BF16 && t_dtype != OFQ_F32,
                OFQ_ERR_BAD_DTYPE);
  OFQ_RETURN_IF(outer < 0 || group_size <= 0 || inner <= 0, OFQ_ERR_BAD_SHAPE);
  // codes are packed along the last axis, so its unpacked length must be a multiple of 8/bits
  const int64_t last = inner == 1 ? group_size : inner;
  OFQ_RETURN_IF(last % (8 / num_bits) != 0, OFQ_ERR_BAD_SHAPE);
  if (outer == 0) return OFQ_OK;
  OFQ_RETURN_IF(in == nullptr || scale == nullptr || out == nullptr, OFQ_ERR_NULL_POINTER);
  OFQ_RETURN_IF((symmetric != 0) != (zero == nullptr), OFQ_ERR_NULL_POINTER);
  OFQ_RETURN_IF(!ofq_aligned16(in) || !ofq_aligned16(out) || !ofq_aligned16(scale)
                    || !ofq_aligned16(zero),
                OFQ_ERR_MISALIGNED);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool sg = in_dtype == OFQ_I8;
  const bool sym = symmetric != 0;
  switch (t_dtype) {
    case OFQ_F16:
      return ofq::dispatch<ofq::f16>(st, in, scale, zero, out, sg, num_bits, sym, outer,
                                     group_size, inner);
    case OFQ_BF16:
      return ofq::dispatch<ofq::bf16>(st, in, scale, zero, out, sg, num_bits, sym, outer,
                                      group_size, inner);
    default:
      return ofq::dispatch<float>(st, in, scale, zero, out, sg, num_bits, sym, outer, group_size,
                                  inner);
  }
}
