/*
 * CPU oracle for OneFlow's quantized-inference op family.
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain scalar C, the arithmetic of the
 * reference kernels so that the HIP kernels can be checked against it.  Nothing that ships
 * (the HIP library, its C ABI, the Python/C++ host layers) may call into this file; only the
 * test-suite, the smoke check and the benchmark's CPU-baseline leg load it.
 *
 * Every function names the reference lines it follows (paths relative to the OneFlow tree).
 * Compile with -ffp-contract=off: every `*` and `+` below is meant to round on its own.
 *
 * Pinning status (what independent evidence fixes each function; see tests/test_oracle_*.py):
 *   min_max_observer / quantization / fake_quantization (f32):
 *       pinned by a 12-row known-answer table (tests/golden/ref_cpu_known_answers.json) that a
 *       test rebuilds in exact rational arithmetic with one fp32 rounding per operation of
 *       min_max_observer_kernel.cpp:22-46 / quantization_kernel.cpp:22-48, symmetric and affine,
 *       by round-half-even tie vectors, and by invariants (|x/s - code| <= 0.5, row absmax ->
 *       +-(2^(b-1)-1), codes in range).
 *   groupwise_dequantize:
 *       pinned by brute force over every code value against exact rational arithmetic rounded
 *       once per operation (fractions + numpy.float16 / bit-level bf16), by s=1,z=0 identity and
 *       by the int4 nibble order of the reference test's packer.
 *   fused_linear (dequantize -> matmul, fp32 accumulate):
 *       pinned by the integer special case (all scales 1 -> exact integer GEMV), M-invariance and
 *       an independent numpy float64 composition within fp32-accumulation error.
 *   layer_norm_min_max_observer, matmul_quant:
 *       the reference holds no such op (only the env-var name ONEFLOW_MLIR_GROUP_MATMUL_QUANT);
 *       semantics are defined by composition of reference rules.  The LayerNorm half is pinned
 *       on its rule (layer_norm_gpu_kernel.cu:61-68) bit for bit in fp16 and bf16: rows with
 *       exactly known mean and variance, expected bits built with numpy / torch casts as
 *       T(T(T(n) * gamma) + beta), and three plausible wrong rounding orders shown to differ;
 *       matmul_quant by an exact int64 GEMM.  As fused ops they have no counterpart to compare
 *       with: PARITY OF THE COMPOSITION WITH THE REFERENCE UNPINNED for these two.
 *   groupwise_quantize, moving_average_min_max_observer:
 *       pinned against an independent numpy restatement of the reference test's quantiser and
 *       closed forms / hand-written fp32 step sequences.
 *   skip_layer_norm input (skip_layer_norm_min_max_observer):
 *       pinned bit for bit on the reference test's own composition (add bias, add skip*alpha,
 *       layer_norm) evaluated in T with numpy and fed to the LayerNorm oracle above.
 *   glu_gate:
 *       'none' / 'relu' / sigmoid(0) exact closed forms; sigmoid, silu, gelu, fast_gelu against
 *       float64 evaluations (scipy erf, numpy exp / tanh) to one rounding of T.  The reference's
 *       architecture-dependent fp16 fast_gelu (tanh approximation instruction) is not restated:
 *       PARITY UNPINNED for fast_gelu in fp16 against that variant.
 *   double precision observer/quantization paths and the "cambricon" formula:
 *       same code as f32 through a macro; cambricon pinned only by closed-form powers of two.
 */
#include <fenv.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "ofq_oracle.h"

/* ------------------------------------------------------------------------------------------
 * Software fp16 / bf16 conversions (round-to-nearest-even), so the oracle needs no compiler
 * half type.  Arithmetic in T is done as: widen to fp32, one fp32 operation, round to T.  For
 * +,-,* this equals a correctly rounded T operation because fp32 carries 24 >= 2p+2 significand
 * bits for p = 11 (fp16) and p = 8 (bf16).
 * ---------------------------------------------------------------------------------------- */
static inline uint32_t f32_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
static inline float bits_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}

float ofq_ref_half_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1Fu;
  uint32_t man = h & 0x3FFu;
  if (exp == 0) {
    if (man == 0) return bits_f32(sign);
    /* subnormal: normalise */
    int e = -1;
    do {
      man <<= 1;
      ++e;
    } while ((man & 0x400u) == 0);
    man &= 0x3FFu;
    return bits_f32(sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13));
  }
  if (exp == 31) return bits_f32(sign | 0x7F800000u | (man << 13));
  return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

uint16_t ofq_ref_float_to_half(float f) {
  const uint32_t u = f32_bits(f);
  const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  const uint32_t abs = u & 0x7FFFFFFFu;
  if (abs >= 0x7F800000u) { /* inf / nan */
    return (uint16_t)(sign | 0x7C00u | ((abs > 0x7F800000u) ? (0x200u | ((abs >> 13) & 0x3FFu)) : 0));
  }
  if (abs >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u); /* rounds to >= 65520 -> inf */
  if (abs < 0x33000001u) return sign;                          /* <= 2^-25 -> +-0 */
  int32_t exp = (int32_t)(abs >> 23) - 127;
  uint32_t man = (abs & 0x7FFFFFu) | 0x800000u;
  int shift;
  uint32_t half_exp;
  if (exp < -14) { /* subnormal result */
    shift = 13 + (-14 - exp);
    half_exp = 0;
  } else {
    shift = 13;
    half_exp = (uint32_t)(exp + 15);
  }
  uint32_t q = man >> shift;
  const uint32_t rem = man & ((1u << shift) - 1u);
  const uint32_t halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (q & 1u))) ++q;
  uint32_t out;
  if (half_exp == 0) {
    out = q; /* may carry into exponent 1, which is the right encoding */
  } else {
    out = ((half_exp - 1) << 10) + q; /* q includes the hidden bit (0x400); carry propagates */
  }
  return (uint16_t)(sign | out);
}

/* bf16 rule of the reference host type: oneflow/core/common/bfloat16.h:50-71 */
uint16_t ofq_ref_float_to_bf16(float f) {
  if (isnan(f)) return 0x7FC0u;
  const uint32_t u = f32_bits(f);
  const uint32_t bias = ((u >> 16) & 1u) + 0x7FFFu;
  return (uint16_t)((u + bias) >> 16);
}
float ofq_ref_bf16_to_float(uint16_t b) { return bits_f32((uint32_t)b << 16); }

static inline float t_load(const void* p, int64_t i, int t) {
  switch (t) {
    case OFQ_REF_F16: return ofq_ref_half_to_float(((const uint16_t*)p)[i]);
    case OFQ_REF_BF16: return ofq_ref_bf16_to_float(((const uint16_t*)p)[i]);
    default: return ((const float*)p)[i];
  }
}
/* round an fp32 value to T and return it widened again */
static inline float t_round(float v, int t) {
  switch (t) {
    case OFQ_REF_F16: return ofq_ref_half_to_float(ofq_ref_float_to_half(v));
    case OFQ_REF_BF16: return ofq_ref_bf16_to_float(ofq_ref_float_to_bf16(v));
    default: return v;
  }
}
static inline void t_store(void* p, int64_t i, float v, int t) {
  switch (t) {
    case OFQ_REF_F16: ((uint16_t*)p)[i] = ofq_ref_float_to_half(v); break;
    case OFQ_REF_BF16: ((uint16_t*)p)[i] = ofq_ref_float_to_bf16(v); break;
    default: ((float*)p)[i] = v; break;
  }
}

/* ------------------------------------------------------------------------------------------
 * min_max_observer, quantization, fake_quantization -- float and double through one macro.
 * ---------------------------------------------------------------------------------------- */
#define OFQ_DEFINE_QUANT_FAMILY(T, SFX, NEARBYINT, ROUND, FLOOR, LOG2, FABS)                       \
  /* GenQuantScale{Symmetric,Affine,Cambricon}: min_max_observer_kernel.cpp:22-58 */               \
  static void gen_scale_##SFX(const T* in, int64_t n, int bits, int scheme, int formula,           \
                              T* scale, T* zero_point) {                                          \
    T in_max = in[0], in_min = in[0];                                                              \
    for (int64_t i = 1; i < n; ++i) {                                                              \
      /* std::max_element / std::min_element semantics: strict '<' comparisons */                  \
      if (in_max < in[i]) in_max = in[i];                                                          \
      if (in[i] < in_min) in_min = in[i];                                                          \
    }                                                                                              \
    if (formula == OFQ_REF_FORMULA_CAMBRICON) {                                                    \
      T a = FABS(in_max), b = FABS(in_min);                                                        \
      T m = a < b ? b : a; /* std::max(a,b) */                                                     \
      *scale = FLOOR(LOG2(m)) - (T)(bits - 2);                                                     \
      *zero_point = 0;                                                                             \
    } else if (scheme == OFQ_REF_SCHEME_SYMMETRIC) {                                               \
      T a = FABS(in_max), b = FABS(in_min);                                                        \
      T m = a < b ? b : a;                                                                         \
      T denominator = (T)pow(2.0, bits - 1) - 1;                                                   \
      *scale = m / denominator;                                                                    \
      *zero_point = 0;                                                                             \
    } else {                                                                                       \
      T denominator = (T)pow(2.0, bits) - 1;                                                       \
      *scale = (in_max - in_min) / denominator;                                                    \
      *zero_point = -NEARBYINT(in_min / (*scale));                                                 \
    }                                                                                              \
  }                                                                                                \
  /* CpuMinMaxObserverKernel::Compute: min_max_observer_kernel.cpp:67-114 */                       \
  int ofq_ref_min_max_observer_##SFX(const T* in, int64_t elem_cnt, int64_t outer, int bits,       \
                                     int scheme, int formula, T* scale, T* zero_point) {          \
    if (formula == OFQ_REF_FORMULA_CAMBRICON && outer != 1) return -1;                             \
    if (outer <= 0 || elem_cnt % outer != 0) return -1;                                            \
    const int64_t inner = elem_cnt / outer;                                                        \
    for (int64_t c = 0; c < outer; ++c)                                                            \
      gen_scale_##SFX(in + c * inner, inner, bits, scheme, formula, scale + c, zero_point + c);    \
    return 0;                                                                                      \
  }                                                                                                \
  /* QuantizationPerLayer{Symmetric,Affine,Cambricon}: quantization_kernel.cpp:22-62;            \
   * FakeQuantizationPerLayer*: fake_quantization_kernel.cpp:22-64.                              \
   * zp_mode 0 = CPU rule (zero point rounded to uint8 first, quantization_kernel.cpp:41),       \
   * zp_mode 1 = CUDA rule (float zero point as is, quantization_kernel.cu:65-67). */            \
  static void quant_panel_##SFX(const T* in, T scale, T zp, int bits, int scheme, int formula,     \
                                int zp_mode, int fake, int64_t n, T* out) {                       \
    if (formula == OFQ_REF_FORMULA_CAMBRICON) {                                                    \
      T upper = (T)pow(2.0, bits - 1) - 1;                                                         \
      T lower = -upper - 1;                                                                        \
      T s = (T)pow(2.0, (int32_t)scale);                                                           \
      for (int64_t i = 0; i < n; ++i) {                                                            \
        T o = NEARBYINT(in[i] / s);                                                                \
        o = o > upper ? upper : o;                                                                 \
        o = o < lower ? lower : o;                                                                 \
        out[i] = fake ? o * s : o;                                                                 \
      }                                                                                            \
    } else if (scheme == OFQ_REF_SCHEME_SYMMETRIC) {                                               \
      T upper = (T)pow(2.0, bits - 1) - 1;                                                         \
      T lower = -upper - 1;                                                                        \
      for (int64_t i = 0; i < n; ++i) {                                                            \
        T o = NEARBYINT(in[i] / scale);                                                            \
        o = o > upper ? upper : o;                                                                 \
        o = o < lower ? lower : o;                                                                 \
        out[i] = fake ? o * scale : o;                                                             \
      }                                                                                            \
    } else {                                                                                       \
      T upper = (T)pow(2.0, bits) - 1;                                                             \
      T lower = 0;                                                                                 \
      if (zp_mode == 0) {                                                                          \
        uint8_t zp8 = (uint8_t)ROUND(zp);                                                          \
        for (int64_t i = 0; i < n; ++i) {                                                          \
          T o = NEARBYINT(in[i] / scale + zp8);                                                    \
          o = o > upper ? upper : o;                                                               \
          o = o < lower ? lower : o;                                                               \
          out[i] = fake ? (o - zp8) * scale : o;                                                   \
        }                                                                                          \
      } else {                                                                                     \
        for (int64_t i = 0; i < n; ++i) {                                                          \
          T o = NEARBYINT(in[i] / scale + zp);                                                     \
          o = o > upper ? upper : o;                                                               \
          o = o < lower ? lower : o;                                                               \
          out[i] = fake ? (o - zp) * scale : o;                                                    \
        }                                                                                          \
      }                                                                                            \
    }                                                                                              \
  }                                                                                                \
  /* Cpu(Fake)QuantizationKernel::Compute: quantization_kernel.cpp:71-120 (per-channel iff       \
   * scale has more than one element; round-to-nearest set around the loops :86-87,119). */      \
  int ofq_ref_quantization_##SFX(const T* in, const T* scale, const T* zero_point, T* out,         \
                                 int64_t elem_cnt, int64_t scale_size, int64_t shape0, int bits,  \
                                 int scheme, int formula, int zp_mode, int fake) {                \
    const int saved = fegetround();                                                                \
    fesetround(FE_TONEAREST);                                                                      \
    int64_t outer = 1, inner = elem_cnt;                                                           \
    if (formula != OFQ_REF_FORMULA_CAMBRICON && scale_size > 1) {                                  \
      if (shape0 <= 0 || elem_cnt % shape0 != 0 || scale_size != shape0) {                         \
        fesetround(saved);                                                                         \
        return -1;                                                                                 \
      }                                                                                            \
      outer = shape0;                                                                              \
      inner = elem_cnt / shape0;                                                                   \
    }                                                                                              \
    for (int64_t c = 0; c < outer; ++c)                                                            \
      quant_panel_##SFX(in + c * inner, scale[c], zero_point ? zero_point[c] : 0, bits, scheme,    \
                        formula, zp_mode, fake, inner, out + c * inner);                          \
    fesetround(saved);                                                                             \
    return 0;                                                                                      \
  }

OFQ_DEFINE_QUANT_FAMILY(float, f32, nearbyintf, roundf, floorf, log2f, fabsf)
OFQ_DEFINE_QUANT_FAMILY(double, f64, nearbyint, round, floor, log2, fabs)

/* ------------------------------------------------------------------------------------------
 * groupwise_dequantize
 * ---------------------------------------------------------------------------------------- */
/* Cast<uint8_t|int8_t, Dst>: groupwise_quantization_kernels.cu:46-87.  For 4-bit codes element
 * 2i is the HIGH nibble of byte i and element 2i+1 the LOW nibble; an int8 container
 * sign-extends each nibble (arithmetic shifts). */
static inline int code_at(const uint8_t* q, int64_t idx, int bits, int is_signed) {
  if (bits == 8) return is_signed ? (int)(int8_t)q[idx] : (int)q[idx];
  const uint8_t byte = q[idx >> 1];
  if (is_signed) {
    const int8_t s = (int8_t)byte;
    if ((idx & 1) == 0) return (int)(int8_t)(s >> 4);
    int8_t lo = (int8_t)(uint8_t)(byte << 4);
    return (int)(int8_t)(lo >> 4);
  }
  return (idx & 1) == 0 ? (byte >> 4) : (byte & 0xF);
}

/* zero term of a group: groupwise_quantization_kernels.cu:186-198 and :282-293 */
static inline float group_zero(const void* zero, int64_t zi, float scale, int bits, int symmetric,
                               int is_signed, int t) {
  if (!symmetric) return t_load(zero, zi, t);
  if (is_signed) return 0.0f;
  return t_round(-(float)((1 << (bits - 1)) - 1) * scale, t); /* -T(2^(b-1)-1) * scale, in T */
}

/* moving_average_min_max_observer: GenQuantScalePerLayer{Symmetric,Affine,Cambricon},
 * oneflow/user/kernels/moving_average_min_max_observer_kernel.cpp:22-107.  `T * float` widens
 * the float; `(1 - momentum)` is a float expression; the affine zero point uses std::round
 * (half away from zero, :78). */
#define OFQ_DEFINE_MOVING_AVERAGE(T, SUFFIX, ROUND, FLOOR, LOG2, FABS)                            \
  int ofq_ref_moving_average_min_max_observer_##SUFFIX(                                            \
      const T* in, int64_t elem_cnt, int64_t current_train_step, int64_t stop_update_after_iters, \
      int training, int bits, int scheme, int formula, float momentum, T* moving_max,             \
      T* moving_min, T* scale, T* zero_point) {                                                   \
    if (elem_cnt < 1) return -1;                                                                  \
    if (current_train_step <= stop_update_after_iters && training) {                              \
      T in_max = in[0], in_min = in[0];                                                           \
      for (int64_t i = 1; i < elem_cnt; ++i) {                                                    \
        if (in[i] > in_max) in_max = in[i];                                                       \
        if (in[i] < in_min) in_min = in[i];                                                       \
      }                                                                                           \
      const int symmetric_like = formula == OFQ_REF_FORMULA_CAMBRICON                             \
                                 || scheme == OFQ_REF_SCHEME_SYMMETRIC;                           \
      if (symmetric_like) {                                                                       \
        const T a = FABS(in_max), b = FABS(in_min);                                               \
        in_max = a < b ? b : a;                                                                   \
      }                                                                                           \
      const T mm = *moving_max;                                                                   \
      if (mm == 0) {                                                                              \
        *moving_max = in_max;                                                                     \
      } else {                                                                                    \
        const T p0 = mm * momentum;                                                               \
        const T p1 = in_max * (1 - momentum);                                                     \
        *moving_max = p0 + p1;                                                                    \
      }                                                                                           \
      if (symmetric_like) {                                                                       \
        *moving_min = *moving_max;                                                                \
      } else {                                                                                    \
        const T mn = *moving_min;                                                                 \
        if (mn == 0) {                                                                            \
          *moving_min = in_min;                                                                   \
        } else {                                                                                  \
          const T p0 = mn * momentum;                                                             \
          const T p1 = in_min * (1 - momentum);                                                   \
          *moving_min = p0 + p1;                                                                  \
        }                                                                                         \
      }                                                                                           \
    }                                                                                             \
    if (formula == OFQ_REF_FORMULA_CAMBRICON) {                                                   \
      *scale = FLOOR(LOG2(*moving_max)) - (T)(bits - 2);                                          \
      *zero_point = 0;                                                                            \
    } else if (scheme == OFQ_REF_SCHEME_SYMMETRIC) {                                              \
      const T denominator = (T)pow(2.0, bits - 1) - 1;                                            \
      *scale = (*moving_max) / denominator;                                                       \
      *zero_point = 0;                                                                            \
    } else {                                                                                      \
      const T denominator = (T)pow(2.0, bits) - 1;                                                \
      *scale = ((*moving_max) - (*moving_min)) / denominator;                                     \
      *zero_point = -ROUND((*moving_min) / (*scale));                                             \
    }                                                                                             \
    return 0;                                                                                     \
  }
OFQ_DEFINE_MOVING_AVERAGE(float, f32, roundf, floorf, log2f, fabsf)
OFQ_DEFINE_MOVING_AVERAGE(double, f64, round, floor, log2, fabs)

/* Weight quantiser + packer: the `_quantize` / `_pack_int8_to_int4` helpers of the reference's
 * own test, python/oneflow/test/modules/test_groupwise_quantization.py:26-81, restated.  All
 * arithmetic is fp32 (`x.float()`), `flow.round` rounds half to even, scale and zero are cast to
 * T at the end; the codes are computed with the UNROUNDED fp32 scale.
 *   symmetric : scale = absmax / (2^(b-1)-1);  q = rint(x / scale + offset),
 *               offset = 2^(b-1)-1 for a uint8 container, 0 for int8
 *   asymmetric: scale = (max - min) / (2^b - 1); q = rint((x - min) / scale); zero = min
 * x is [n,k]; groups of `group_size` along axis `group_dim`; 4-bit codes are packed along k,
 * element 2i in the high nibble.  A group whose scale is 0 (all elements equal / zero) would be
 * 0/0 in the reference helper; here its codes are defined as `offset` (symmetric) or 0. */
int ofq_ref_groupwise_quantize(const void* x, void* q, void* scale, void* zero, int t,
                               int q_is_signed, int bits, int symmetric, int group_dim,
                               int64_t group_size, int64_t n, int64_t k) {
  if ((bits != 4 && bits != 8) || (group_dim != 0 && group_dim != 1) || group_size <= 0) return -1;
  if (!symmetric && (q_is_signed || zero == NULL)) return -1;
  if (bits == 4 && (k % 2) != 0) return -1;
  const int64_t dim = group_dim == 0 ? n : k;
  if (dim % group_size != 0) return -1;
  const int64_t outer = group_dim == 0 ? 1 : n;
  const int64_t groups = dim / group_size;
  const int64_t inner = group_dim == 0 ? k : 1;
  uint8_t* qb = (uint8_t*)q;
  const float signed_max = (float)((1 << (bits - 1)) - 1);
  const float unsigned_max = (float)((1 << bits) - 1);
  for (int64_t o = 0; o < outer; ++o)
    for (int64_t g = 0; g < groups; ++g)
      for (int64_t i = 0; i < inner; ++i) {
        float mn = 0.0f, mx = 0.0f, amax = 0.0f;
        for (int64_t j = 0; j < group_size; ++j) {
          const float v = t_load(x, ((o * groups + g) * group_size + j) * inner + i, t);
          if (j == 0 || v < mn) mn = v;
          if (j == 0 || v > mx) mx = v;
          if (fabsf(v) > amax) amax = fabsf(v);
        }
        const float sc = symmetric ? amax / signed_max : (mx - mn) / unsigned_max;
        const float offset = symmetric ? (q_is_signed ? 0.0f : signed_max) : 0.0f;
        t_store(scale, (o * groups + g) * inner + i, sc, t);
        if (!symmetric) t_store(zero, (o * groups + g) * inner + i, mn, t);
        for (int64_t j = 0; j < group_size; ++j) {
          const int64_t idx = ((o * groups + g) * group_size + j) * inner + i;
          const float v = t_load(x, idx, t);
          float r;
          if (sc == 0.0f) {
            r = offset;
          } else if (symmetric) {
            const float d = v / sc;
            r = nearbyintf(d + offset);
          } else {
            const float d = v - mn;
            r = nearbyintf(d / sc);
          }
          const int code = (int)r;
          if (bits == 8) {
            qb[idx] = (uint8_t)code;
          } else {
            const uint8_t nib = (uint8_t)code & 0xF;
            if ((idx & 1) == 0) {
              qb[idx >> 1] = (uint8_t)((qb[idx >> 1] & 0x0F) | (nib << 4));
            } else {
              qb[idx >> 1] = (uint8_t)((qb[idx >> 1] & 0xF0) | nib);
            }
          }
        }
      }
  return 0;
}

/* Dequantize3D / DequantizeInnerSize1: groupwise_quantization_kernels.cu:170-203, :275-299;
 * element arithmetic InplaceFma(Scalar) :97-103,123-130: elem * scale + zero, each op in T.
 * View: out[outer][group_size][inner]; scale/zero[outer][inner]; codes packed along the last
 * axis of the ORIGINAL tensor (the flat unpacked index is what is halved for 4-bit). */
int ofq_ref_groupwise_dequantize(const void* in, const void* scale, const void* zero, void* out,
                                 int in_is_signed, int t, int bits, int symmetric, int64_t outer,
                                 int64_t group_size, int64_t inner) {
  if (bits != 4 && bits != 8) return -1;
  if (!symmetric && zero == NULL) return -1;
  for (int64_t o = 0; o < outer; ++o) {
    for (int64_t i = 0; i < inner; ++i) {
      const float s = t_load(scale, o * inner + i, t);
      const float z = group_zero(zero, o * inner + i, s, bits, symmetric, in_is_signed, t);
      for (int64_t g = 0; g < group_size; ++g) {
        const int64_t idx = (o * group_size + g) * inner + i;
        const float q = (float)code_at((const uint8_t*)in, idx, bits, in_is_signed);
        const float prod = t_round(q * s, t);
        t_store(out, idx, prod + z, t);
      }
    }
  }
  return 0;
}

/* ------------------------------------------------------------------------------------------
 * fused_linear_with_groupwise_quantized_weight: the composition the reference functor runs for
 * m > 8 and its test uses as the expected value (functional/impl/quantization.cpp:341-350,
 * test_groupwise_quantization.py:161-175): dequantize in T, then x @ w~^T accumulated in a wide
 * type, + bias, rounded once to T.  acc_mode 0: fp32 accumulation in k order (the stated
 * parity contract); 1: fp64 accumulation (used to bound the accumulation-order error).
 * Shapes: x[m,k], w[n, k*bits/8], scale/zero [n, k/g] (group_dim 1) or [n/g, k] (group_dim 0),
 * bias[n] or NULL, out[m,n]   (groupwise_quantization_kernels.cu:760-839).
 * ---------------------------------------------------------------------------------------- */
int ofq_ref_fused_linear(const void* x, const void* w, const void* scale, const void* zero,
                         const void* bias, void* out, int w_is_signed, int t, int bits,
                         int symmetric, int group_dim, int64_t group_size, int64_t m, int64_t n,
                         int64_t k, int acc_mode) {
  if (bits != 4 && bits != 8) return -1;
  if (group_dim != 0 && group_dim != 1) return -1;
  if (!symmetric && zero == NULL) return -1;
  float* wrow = (float*)malloc(sizeof(float) * (size_t)k);
  float* xf = (float*)malloc(sizeof(float) * (size_t)(m * k));
  if (!wrow || !xf) {
    free(wrow);
    free(xf);
    return -2;
  }
  for (int64_t i = 0; i < m * k; ++i) xf[i] = t_load(x, i, t);
  const int64_t groups_per_row = group_dim == 1 ? k / group_size : 0;
  for (int64_t j = 0; j < n; ++j) {
    for (int64_t kk = 0; kk < k; ++kk) {
      const int64_t si = group_dim == 1 ? j * groups_per_row + kk / group_size
                                        : (j / group_size) * k + kk;
      const float s = t_load(scale, si, t);
      const float z = group_zero(zero, si, s, bits, symmetric, w_is_signed, t);
      const float q = (float)code_at((const uint8_t*)w, j * k + kk, bits, w_is_signed);
      wrow[kk] = t_round(t_round(q * s, t) + z, t);
    }
    for (int64_t i = 0; i < m; ++i) {
      const float* xi = xf + i * k;
      float r;
      if (acc_mode == 0) {
        float acc = 0.0f;
        for (int64_t kk = 0; kk < k; ++kk) acc += xi[kk] * wrow[kk];
        if (bias) acc += t_load(bias, j, t);
        r = acc;
      } else {
        double acc = 0.0;
        for (int64_t kk = 0; kk < k; ++kk) acc += (double)xi[kk] * (double)wrow[kk];
        if (bias) acc += (double)t_load(bias, j, t);
        r = (float)acc;
      }
      t_store(out, i * n + j, r, t);
    }
  }
  free(wrow);
  free(xf);
  return 0;
}

/* ------------------------------------------------------------------------------------------
 * fused_layer_norm_min_max_observer (op absent from the reference; composed from its rules).
 * LayerNorm: per-row mean / variance, var = max(M2/n, 0), inv = rsqrt(var + eps)
 *   (core/cuda/layer_norm.cuh:212-233, :377-380); the normalised value is cast to T BEFORE the
 *   affine, which is then done in T: y = T(T(n_i * gamma) + beta)
 *   (user/kernels/layer_norm_gpu_kernel.cu:40-70).  Mean and variance are taken here in double
 *   (two-pass) and rounded to fp32; the reference accumulates them in fp32 in a thread-dependent
 *   order, so the last fp32 bit of mean/inv is not defined by it.
 * Observer: per-tensor symmetric, scale = absmax(y) / (2^(b-1)-1) as one fp32 divide
 *   (min_max_observer_kernel.cpp:22-34 applied to the T-rounded y), zero_point = 0.
 * ---------------------------------------------------------------------------------------- */
/* The input of the normalisation with the optional residual of skip_layer_norm
 * (user/kernels/skip_layer_norm_kernel.cu:36-67): (x + bias[c]) + skip * T(alpha), every
 * operation in T; an absent bias or skip enters as zero, exactly as there. */
static float skip_input(const void* x, const void* bias, const void* skip, float alpha_t,
                        int64_t r, int64_t c, int64_t cols, int t, int with_skip) {
  const float xv = t_load(x, r * cols + c, t);
  if (!with_skip) return xv;
  const float bv = bias ? t_load(bias, c, t) : 0.0f;
  const float sv = skip ? t_load(skip, r * cols + c, t) : 0.0f;
  const float a = t_round(xv + bv, t);
  const float b = t_round(sv * alpha_t, t);
  return t_round(a + b, t);
}

static int layer_norm_observer_impl(const void* x, const void* bias, const void* skip,
                                    double alpha, int with_skip, const void* gamma,
                                    const void* beta, void* y, float* scale, float* zero_point,
                                    int64_t rows, int64_t cols, double eps, int t, int bits) {
  float absmax = 0.0f;
  const float alpha_t = t_round((float)alpha, t);
  for (int64_t r = 0; r < rows; ++r) {
    double sum = 0.0;
    for (int64_t c = 0; c < cols; ++c)
      sum += (double)skip_input(x, bias, skip, alpha_t, r, c, cols, t, with_skip);
    const double mean = sum / (double)cols;
    double m2 = 0.0;
    for (int64_t c = 0; c < cols; ++c) {
      const double d = (double)skip_input(x, bias, skip, alpha_t, r, c, cols, t, with_skip) - mean;
      m2 += d * d;
    }
    double var = m2 / (double)cols;
    if (var < 0.0) var = 0.0;
    const float mean_f = (float)mean;
    const float inv_f = (float)(1.0 / sqrt(var + eps));
    for (int64_t c = 0; c < cols; ++c) {
      const float xin = skip_input(x, bias, skip, alpha_t, r, c, cols, t, with_skip);
      const float xn = t_round((xin - mean_f) * inv_f, t);
      float v = xn;
      /* layer_norm_gpu_kernel.cu:46-59,63-64: with either of gamma / beta present both
       * operations run, the absent operand being 1 or 0 (so -0 + 0 gives +0) */
      if (gamma || beta) {
        v = t_round(v * (gamma ? t_load(gamma, c, t) : 1.0f), t);
        v = t_round(v + (beta ? t_load(beta, c, t) : 0.0f), t);
      }
      t_store(y, r * cols + c, v, t);
      const float a = fabsf(t_round(v, t));
      if (a > absmax) absmax = a;
    }
  }
  const float denominator = (float)pow(2.0, bits - 1) - 1;
  *scale = absmax / denominator;
  *zero_point = 0.0f;
  return 0;
}

int ofq_ref_layer_norm_min_max_observer(const void* x, const void* gamma, const void* beta,
                                        void* y, float* scale, float* zero_point, int64_t rows,
                                        int64_t cols, double eps, int t, int bits) {
  return layer_norm_observer_impl(x, NULL, NULL, 0.0, 0, gamma, beta, y, scale, zero_point, rows,
                                  cols, eps, t, bits);
}

/* fused_skip_layer_norm_min_max_observer: the same with the input of skip_layer_norm. */
int ofq_ref_skip_layer_norm_min_max_observer(const void* x, const void* bias, const void* skip,
                                             double alpha, const void* gamma, const void* beta,
                                             void* y, float* scale, float* zero_point,
                                             int64_t rows, int64_t cols, double eps, int t,
                                             int bits) {
  return layer_norm_observer_impl(x, bias, skip, alpha, 1, gamma, beta, y, scale, zero_point,
                                  rows, cols, eps, t, bits);
}

/* ------------------------------------------------------------------------------------------
 * The gating of fused_glu (user/kernels/fused_glu_kernel.cu:303-347): per element
 *   y = hidden_state * act(gate), hidden_state = matmul_wx[r*stride + c],
 *   gate = matmul_vx[r*stride + c], both operations in T.  For the 16-bit types the activation
 *   is the fp32 functor applied to the widened value and rounded back
 *   (ep/cuda/primitive/unary_functor.cuh:449-464,522-570); fp32 forms:
 *   ep/common/primitive/unary_functor.h:146-170,477-484 (relu, silu, sigmoid),
 *   ep/cuda/primitive/unary_functor.cuh:31-58 (gelu, fast_gelu).  fast_gelu follows the generic
 *   form for every T (the reference has an architecture-dependent fp16 variant, :100-136).
 * act: 0 none, 1 sigmoid, 2 relu, 3 gelu, 4 fast_gelu, 5 silu.
 * ---------------------------------------------------------------------------------------- */
static float glu_activation(float v, int act) {
  switch (act) {
    case 1: return 1.0f / (1.0f + expf(-v));
    case 2: return v <= 0.0f ? 0.0f : v;
    case 3: return 0.5f * v * (1.0f + erff(0.70710678118654752440f * v));
    case 4: {
      const float alpha = 0.7978845608028654f;
      const float beta = 0.044714998453855515f;
      const float tanh_in = alpha * (v + beta * v * v * v);
      return 0.5f * v * (1.0f + tanhf(tanh_in));
    }
    case 5: return v / (1.0f + expf(-v));
    default: return v;
  }
}

int ofq_ref_glu_gate(const void* matmul_wx, const void* matmul_vx, void* y, int64_t m, int64_t n,
                     int64_t stride, int t, int act) {
  if (act < 0 || act > 5) return 1;
  for (int64_t r = 0; r < m; ++r) {
    for (int64_t c = 0; c < n; ++c) {
      const float h = t_load(matmul_wx, r * stride + c, t);
      const float g = t_load(matmul_vx, r * stride + c, t);
      const float a = t_round(glu_activation(g, act), t);
      t_store(y, r * n + c, h * a, t);
    }
  }
  return 0;
}

/* quantization with a low-precision input and int8 codes (the dynamic activation path): the
 * same rule as QuantizationPerLayerSymmetric (quantization_kernel.cpp:22-33) evaluated in fp32
 * on the widened input, codes narrowed to int8 (exact: the clamp keeps them in [-128,127]). */
int ofq_ref_quantize_to_int8(const void* in, const float* scale, int8_t* out, int64_t elem_cnt,
                             int64_t scale_size, int64_t shape0, int t, int bits) {
  const int saved = fegetround();
  fesetround(FE_TONEAREST);
  const float upper = (float)pow(2.0, bits - 1) - 1;
  const float lower = -upper - 1;
  const int64_t inner = scale_size > 1 ? elem_cnt / shape0 : elem_cnt;
  for (int64_t i = 0; i < elem_cnt; ++i) {
    const float s = scale[scale_size > 1 ? i / inner : 0];
    float o = nearbyintf(t_load(in, i, t) / s);
    o = o > upper ? upper : o;
    o = o < lower ? lower : o;
    out[i] = (o != o) ? 0 : (int8_t)o; /* NaN (0/0 on an all-zero tensor) narrows to 0 */
  }
  fesetround(saved);
  return 0;
}

/* ------------------------------------------------------------------------------------------
 * matmul_quant (op absent from the reference).  a[m,k] int8, b[n,k] int8 (weight layout of
 * fused_matmul_bias: OneFlowUserOps.td:5615-5633), exact int32 accumulation, then
 * out = T( float(acc) * fl32(a_scale * b_scale[n]) (+ float(bias[n])) ).
 * ---------------------------------------------------------------------------------------- */
int ofq_ref_matmul_quant(const int8_t* a, const int8_t* b, const float* a_scale,
                         const float* b_scale, const void* bias, void* out, int t, int64_t m,
                         int64_t n, int64_t k) {
  for (int64_t i = 0; i < m; ++i) {
    for (int64_t j = 0; j < n; ++j) {
      int32_t acc = 0;
      const int8_t* ai = a + i * k;
      const int8_t* bj = b + j * k;
      for (int64_t kk = 0; kk < k; ++kk) acc += (int32_t)ai[kk] * (int32_t)bj[kk];
      const float s = a_scale[0] * b_scale[j];
      float r = (float)acc * s;
      if (bias) r = r + t_load(bias, j, t);
      t_store(out, i * n + j, r, t);
    }
  }
  return 0;
}
