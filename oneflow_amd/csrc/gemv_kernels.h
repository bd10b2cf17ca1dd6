// Device code of the skinny-M (decode) kernels of fused_linear_with_groupwise_quantized_weight.
// Kept in a header so that experiments can instantiate the kernels directly.
#pragma once

#include "ofq_device.h"

namespace ofq {
namespace {

enum { kZeroNone = 0, kZeroSymU = 1, kZeroAsym = 2 };

__device__ __forceinline__ f16x2 as_h2(uint32_t u) { return __builtin_bit_cast(f16x2, u); }
__device__ __forceinline__ uint32_t as_u32(f16x2 h) { return __builtin_bit_cast(uint32_t, h); }

// eight 4-bit codes of `word` as exact fp16 values, in the pair order
// (e1,e5) (e0,e4) (e3,e7) (e2,e6) where e_i is element i of the word (element 0 = high nibble
// of byte 0).
template<bool SIGNED>
__device__ __forceinline__ void unpack4_pairs(uint32_t word, f16x2 (&o)[4]) {
  if (SIGNED) word ^= 0x88888888u;
  const uint32_t w8 = word >> 8;
  const f16 off_lo = SIGNED ? (f16)(-1032.0f) : (f16)(-1024.0f);
  const f16 off_hi = SIGNED ? (f16)(-72.0f) : (f16)(-64.0f);
  const f16x2 ol = {off_lo, off_lo};
  const f16x2 oh = {off_hi, off_hi};
  const f16x2 sixteenth = {(f16)0.0625f, (f16)0.0625f};
  o[0] = as_h2((word & 0x000F000Fu) | 0x64006400u) + ol;
  o[1] = __builtin_elementwise_fma(as_h2((word & 0x00F000F0u) | 0x64006400u), sixteenth, oh);
  o[2] = as_h2((w8 & 0x000F000Fu) | 0x64006400u) + ol;
  o[3] = __builtin_elementwise_fma(as_h2((w8 & 0x00F000F0u) | 0x64006400u), sixteenth, oh);
}

// four 8-bit codes of `word` as exact fp16 values in natural order (b0,b1) (b2,b3)
template<bool SIGNED>
__device__ __forceinline__ void unpack8_pairs(uint32_t word, f16x2 (&o)[2]) {
  if (SIGNED) word ^= 0x80808080u;
  const f16 off = SIGNED ? (f16)(-1152.0f) : (f16)(-1024.0f);
  const f16x2 o2 = {off, off};
  o[0] = as_h2(__builtin_amdgcn_perm(word, 0x64646464u, 0x00050004u)) + o2;
  o[1] = as_h2(__builtin_amdgcn_perm(word, 0x64646464u, 0x00070006u)) + o2;
}

// x permuted to the pair order of unpack4_pairs: [x1,x5,x0,x4,x3,x7,x2,x6]
__device__ __forceinline__ u32x4 permute_x4(u32x4 v) {
  u32x4 r;
  r[0] = __builtin_amdgcn_perm(v[2], v[0], 0x07060302u);  // (x1, x5)
  r[1] = __builtin_amdgcn_perm(v[2], v[0], 0x05040100u);  // (x0, x4)
  r[2] = __builtin_amdgcn_perm(v[3], v[1], 0x07060302u);  // (x3, x7)
  r[3] = __builtin_amdgcn_perm(v[3], v[1], 0x05040100u);  // (x2, x6)
  return r;
}

template<int BITS, bool SIGNED, int ZMODE, int NWAVES, int UNROLL>
__global__ void __launch_bounds__(NWAVES * 64)
gemv_f16_mfma(const f16* __restrict__ x, const uint8_t* __restrict__ w,
              const f16* __restrict__ scale, const f16* __restrict__ zero,
              const f16* __restrict__ bias, f16* __restrict__ out, int M, int N, int K,
              int group_size, int gs_shift) {
  constexpr int CH = BITS == 4 ? 128 : 64;  // k elements per chunk (64 bytes of codes per row)
  constexpr int LK = CH / 4;                // k elements per lane per chunk
  constexpr int NJ = LK / 8;                // MFMAs per chunk
  __shared__ float red[NWAVES][64][4];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int r = lane & 15;
  const int kb = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int n_ld = (n0 + r < N) ? n0 + r : N - 1;  // clamp loads of a partial last tile
  const int nchunks = K / CH;
  const int G = K / group_size;
  const uint8_t* wrow = w + (int64_t)n_ld * ((int64_t)K * BITS / 8);
  const f16* srow = scale + (int64_t)n_ld * G;
  const f16* zrow = ZMODE == kZeroAsym ? zero + (int64_t)n_ld * G : nullptr;
  const bool has_x = r < M;
  const f16* xrow = x + (int64_t)(has_x ? r : 0) * K;

  f32x4 acc0 = {0.f, 0.f, 0.f, 0.f};
  f32x4 acc1 = {0.f, 0.f, 0.f, 0.f};

  for (int c0 = wave; c0 < nchunks; c0 += NWAVES * UNROLL) {
    u32x4 wq[UNROLL];
    u32x4 xv[UNROLL][NJ];
    f16 sv[UNROLL], zv[UNROLL];
    // issue every load of the UNROLL chunks before touching any of them
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = c0 + u * NWAVES;
      const bool valid = c < nchunks;
      const int k0 = (valid ? c : 0) * CH + kb * LK;
      wq[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow + (int64_t)k0 * BITS / 8));
      const int g = gs_shift >= 0 ? (k0 >> gs_shift) : (k0 / group_size);
      sv[u] = srow[g];
      zv[u] = ZMODE == kZeroAsym ? zrow[g] : (f16)0.0f;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const u32x4 t = *reinterpret_cast<const u32x4*>(xrow + k0 + j * 8);
        const u32x4 zero4 = {0u, 0u, 0u, 0u};
        xv[u][j] = (has_x && valid) ? t : zero4;
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const f16 s = sv[u];
      f16 z = zv[u];
      if (ZMODE == kZeroSymU) z = (f16)(-(float)((1 << (BITS - 1)) - 1)) * s;
      const f16x2 s2 = {s, s};
      const f16x2 z2 = {z, z};
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        u32x4 bop;
        u32x4 aop;
        if (BITS == 4) {
          f16x2 p[4];
          unpack4_pairs<SIGNED>(wq[u][j], p);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            f16x2 v = p[e] * s2;
            if (ZMODE != kZeroNone) v = v + z2;
            bop[e] = as_u32(v);
          }
          aop = permute_x4(xv[u][j]);
        } else {
          f16x2 p0[2], p1[2];
          unpack8_pairs<SIGNED>(wq[u][2 * j], p0);
          unpack8_pairs<SIGNED>(wq[u][2 * j + 1], p1);
          f16x2 v[4] = {p0[0] * s2, p0[1] * s2, p1[0] * s2, p1[1] * s2};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (ZMODE != kZeroNone) v[e] = v[e] + z2;
            bop[e] = as_u32(v[e]);
          }
          aop = xv[u][j];
        }
        const f16x8 a8 = __builtin_bit_cast(f16x8, aop);
        const f16x8 b8 = __builtin_bit_cast(f16x8, bop);
        if ((j & 1) == 0) {
          acc0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a8, b8, acc0, 0, 0, 0);
        } else {
          acc1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a8, b8, acc1, 0, 0, 0);
        }
      }
    }
  }
  // lane holds D[m = 4*kb + v][n = n0 + r]
#pragma unroll
  for (int v = 0; v < 4; ++v) red[wave][lane][v] = acc0[v] + acc1[v];
  __syncthreads();
  for (int t = threadIdx.x; t < 256; t += NWAVES * 64) {
    const int l = t >> 2;
    const int v = t & 3;
    float sum = 0.f;
#pragma unroll
    for (int wv = 0; wv < NWAVES; ++wv) sum += red[wv][l][v];
    const int m = 4 * (l >> 4) + v;
    const int n = n0 + (l & 15);
    if (m < M && n < N) {
      if (bias != nullptr) sum += (float)bias[n];
      out[(int64_t)m * N + n] = (f16)sum;
    }
  }
}


// ---------------------------------------------------------------------------------------------
// Fast path: 4-bit symmetric codes in an int8 container (zero term 0), fp16, groups along K with
// 128 | group_size.  A one-shot kernel cannot overlap its arithmetic with the HBM latency it has
// just waited for, and at 8 TB/s the whole chip has only ~20 vector instructions per 32-bit word
// of codes, so the instruction count per word is what this kernel is built around (5, against
// ~17 for gemv_f16_mfma):
//
//  (1) x is permuted into MFMA operand order ONCE per block while the weight loads are in
//      flight, and kept in LDS; the waves then fetch ready-made operands with ds_read_b128
//      (only the lanes of rows m < M read at all).  When M*K is too large for LDS (STAGED =
//      false) each lane loads and permutes the x of its own k-slot instead.
//  (2) The codes are never converted to their integer value.  With u = q+8 (the xor that turns
//      two's complement into offset binary is folded into the mask-and-merge, one v_bitop3) the
//      half 0x6400|u is 1024+u for a low nibble (one ulp of [1024,2048) is 1) and the half
//      0x5400|(u<<4) is 64+u for a high nibble left where it is (one ulp of [64,128) is 1/16, so
//      mantissa bits 4..7 count in units of 1).  One MFMA accumulator collects
//        acc = sum_k x q + 1032 * sum_lo x + 72 * sum_hi x
//      and the constant part `corr` depends on (m, chunk) only: it is computed once per block
//      when x is staged (or with two MFMAs against constant operands when x is not staged).
//      x itself is used as stored (no rescaling, so no range of x is special).
//      All products are exact in fp32; the cancellation is done per chunk of 128 k, where the
//      partial sums are ~1e4 and fp32 resolves 1e-3 of a code unit.  The group scale multiplies
//      the chunk result once (fp32), i.e. w~ = q*s is not rounded to fp16 first: the result is
//      closer to exact arithmetic than the reference kernel's and differs from the
//      dequantize->matmul composition by the rounding of w~ (~3e-4 relative).
//  (3) The 16 x G scales of the block's rows are one contiguous piece of memory: they are
//      fetched with a single coalesced load per block into LDS instead of one 2-byte gather per
//      lane and chunk (which costs as many memory requests as the weights themselves).
//  (4) A wave takes chunks in adjacent pairs, so that both halves of every 128-byte line are
//      requested by the same wave back to back.
//
// LDS layout of x: record (m, chunk) = 256 bytes = [kb 0..3][t 0..3][8 halves], where for the
// 32 k-values of lane-slot kb, t=0/1 hold the k of the low/high nibbles of code words 0,1 and
// t=2/3 those of words 2,3, in the order the nibble masks deliver them: {1,5,3,7,9,13,11,15} and
// {0,4,2,6,8,12,10,14} (+16 for t=2,3).
// ---------------------------------------------------------------------------------------------
constexpr int kGemvMaxUnits = 4;  // 32-byte x units a thread may stage

// (2 v * ceil(2^31 / d)) >> 32 == v / d for v < 2^17 and 1 <= d <= 2^13: the row of x a staging
// unit belongs to, without an integer division per unit
__device__ __forceinline__ uint32_t row_of_inv(int d) { return 0x7FFFFFFFu / (uint32_t)d + 1u; }
__device__ __forceinline__ int row_of(int v, uint32_t inv) {
  return (int)__umulhi((uint32_t)v << 1, inv);
}

// x of one 16-k unit (two 128-bit words, natural order) -> low-nibble operand and high-nibble
// operand
__device__ __forceinline__ void permute_unit(const u32x4 a, const u32x4 b, u32x4& lo, u32x4& hi) {
  lo[0] = __builtin_amdgcn_perm(a[2], a[0], 0x07060302u);  // (x1, x5)
  lo[1] = __builtin_amdgcn_perm(a[3], a[1], 0x07060302u);  // (x3, x7)
  lo[2] = __builtin_amdgcn_perm(b[2], b[0], 0x07060302u);  // (x9, x13)
  lo[3] = __builtin_amdgcn_perm(b[3], b[1], 0x07060302u);  // (x11, x15)
  hi[0] = __builtin_amdgcn_perm(a[2], a[0], 0x05040100u);  // (x0, x4)
  hi[1] = __builtin_amdgcn_perm(a[3], a[1], 0x05040100u);  // (x2, x6)
  hi[2] = __builtin_amdgcn_perm(b[2], b[0], 0x05040100u);  // (x8, x12)
  hi[3] = __builtin_amdgcn_perm(b[3], b[1], 0x05040100u);  // (x10, x14)
}

// 1032 * (sum of the low-nibble x) + 72 * (sum of the high-nibble x) of one permuted unit
// (packed dot products against the two constants: 8 instructions where widening and adding the
// 16 values took 34; every product is exact in fp32)
__device__ __forceinline__ float unit_corr(const u32x4 lo, const u32x4 hi) {
  uint32_t k_lo = 0x64086408u, k_hi = 0x54805480u;  // (1032, 1032), (72, 72), held in registers
  asm volatile("" : "+v"(k_lo), "+v"(k_hi));
  const f16x2 c_lo = as_h2(k_lo), c_hi = as_h2(k_hi);
  float acc = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    acc = __builtin_amdgcn_fdot2(as_h2(lo[i]), c_lo, acc, false);
    acc = __builtin_amdgcn_fdot2(as_h2(hi[i]), c_hi, acc, false);
  }
  return acc;
}

// Pins the widening of a prefetched bias value to the place of use: without the empty asm the
// compiler sinks the conversion (and the wait for every load issued so far) up to the load.
__device__ __forceinline__ f16 bias_at_end(uint16_t raw) {
  uint32_t v = raw;
  asm volatile("" : "+v"(v));
  return __builtin_bit_cast(f16, (uint16_t)v);
}

template<int NWAVES, int UNROLL, bool STAGED>
__global__ void __launch_bounds__(NWAVES * 64)
gemv_w4s_f16(const f16* __restrict__ x, const uint8_t* __restrict__ w,
             const f16* __restrict__ scale, const f16* __restrict__ bias,
             f16* __restrict__ out, int M, int N, int K, int group_size, int cpg_shift) {
  // cpg_shift: log2(group_size / 128) when that is a power of two, else -1 (division per chunk)
  static_assert(UNROLL % 2 == 0, "chunks are taken in pairs");
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  constexpr int NT = NWAVES * 64;
  const int nchunks = K >> 7;
  const uint32_t inv_chunks = row_of_inv(nchunks);
  const int npairs = (nchunks + 1) >> 1;
  const int G = K / group_size;
  // LDS: [reduction NWAVES*64*4 f32][scale tile 16*G halves, padded to 16 B][64 zero bytes]
  //      [x records]
  float* red = reinterpret_cast<float*>(smem);
  f16* sl = reinterpret_cast<f16*>(smem + NWAVES * 64 * 16);
  uint8_t* zrec = smem + NWAVES * 64 * 16 + ((16 * G * 2 + 15) & ~15);  // 64 zero bytes
  uint8_t* xs = zrec + 64;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, kept in an SGPR
  const int r = lane & 15;
  const int kb = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int n_ld = (n0 + r < N) ? n0 + r : N - 1;
  const uint8_t* wrow = w + (int64_t)n_ld * (K >> 1) + kb * 16;
  const bool has_x = r < M;

  // ---- loads that feed LDS are issued first so that they return before the weights ---------
  const int nunits = STAGED ? (M * K) >> 4 : 0;
  u32x4 xu[kGemvMaxUnits][2];
  if (STAGED) {
#pragma unroll
    for (int i = 0; i < kGemvMaxUnits; ++i) {
      if (wave * 64 + i * NT >= nunits) break;  // wave-uniform: nothing left for this wave
      const int u = tid + i * NT;
      if (u < nunits) {
        const u32x4* src = reinterpret_cast<const u32x4*>(x + (int64_t)u * 16);
        xu[i][0] = src[0];
        xu[i][1] = src[1];
      }
    }
  }
  // scale tile: rows n0 .. n0+15 are contiguous; a partial last tile is read element-wise
  const int rows_valid = (N - n0) < 16 ? (N - n0) : 16;
  const int tile_halves = rows_valid * G;
  const f16* stile = scale + (int64_t)n0 * G;
  u32x4 sreg[2];
  bool s_vec[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int e = (tid + i * NT) * 8;  // first half-element of this 16-byte piece
    s_vec[i] = e + 8 <= tile_halves;
    if (s_vec[i]) sreg[i] = *reinterpret_cast<const u32x4*>(stile + e);
  }

  // the bias of the outputs this thread will write at the very end (tid = m * 16 + n)
  // (kept as raw bits: widening it here would wait for every load issued so far)
  uint16_t bias_raw = 0;
  if (bias != nullptr && tid < M * 16 && n0 + (tid & 15) < N) {
    bias_raw = reinterpret_cast<const uint16_t*>(bias)[n0 + (tid & 15)];
  }

  auto chunk_of = [&](int p0, int u) { return 2 * (p0 + (u >> 1) * NWAVES) + (u & 1); };
  u32x4 wq[UNROLL];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const int c = chunk_of(wave, u);
    wq[u] = __builtin_nontemporal_load(
        reinterpret_cast<const u32x4*>(wrow + (c < nchunks ? c : 0) * 64));
  }

  // ---- fill LDS -------------------------------------------------------------------------------
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int e = (tid + i * NT) * 8;
    if (s_vec[i]) {
      *reinterpret_cast<u32x4*>(sl + e) = sreg[i];
    } else if (e < tile_halves) {
      for (int j = e; j < tile_halves && j < e + 8; ++j) sl[j] = stile[j];
    }
  }
  // pieces beyond 2*NT*8 halves (G > NT) are rare; copy them plainly
  for (int e = 2 * NT * 8 + tid; e < tile_halves; e += NT) sl[e] = stile[e];
  if (tid < 16) reinterpret_cast<uint32_t*>(zrec)[tid] = 0u;
  if (STAGED) {
#pragma unroll
    for (int i = 0; i < kGemvMaxUnits; ++i) {
      if (wave * 64 + i * NT >= nunits) break;
      const int u = tid + i * NT;
      if (u < nunits) {
        u32x4 lo, hi;
        permute_unit(xu[i][0], xu[i][1], lo, hi);
        // unit u = (m, chunk, j): j -> kb = j/2, t = 2*(j%2) + {0: lo, 1: hi}; 32 bytes per unit
        // rows of x are skewed by 16 bytes each: the lanes of different m that read the same
        // chunk then hit different LDS bank groups (their records are a multiple of 256 B apart)
        u32x4* dst = reinterpret_cast<u32x4*>(xs + (size_t)u * 32
                                              + row_of(u >> 3, inv_chunks) * 16);
        dst[0] = lo;
        dst[1] = hi;
      }
      // (no correction sums here: the waves get them from the matrix core, see below)
    }
  }
  __syncthreads();

  const uint8_t* xrec = has_x ? xs + (size_t)r * (nchunks * 256 + 16) + kb * 64 : zrec;
  const int xrec_stride = has_x ? 256 : 0;
  const f16* xrow = x + (int64_t)(has_x ? r : 0) * K + kb * 32;
  const f16* slr = sl + r * G;
  const f16 c_lo = (f16)(-1032.0f), c_hi = (f16)(-72.0f);
  const f16x8 kn1032 = {c_lo, c_lo, c_lo, c_lo, c_lo, c_lo, c_lo, c_lo};
  const f16x8 kn72 = {c_hi, c_hi, c_hi, c_hi, c_hi, c_hi, c_hi, c_hi};
  const u32x4 zero4 = {0u, 0u, 0u, 0u};
  f32x4 total = {0.f, 0.f, 0.f, 0.f};

  for (int p0 = wave; p0 < npairs; p0 += NWAVES * (UNROLL / 2)) {
    // prefetch the next group while this one is consumed
    u32x4 wq_next[UNROLL];
    const int pn = p0 + NWAVES * (UNROLL / 2);
    if (pn < npairs) {
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const int c = chunk_of(pn, u);
        wq_next[u] = __builtin_nontemporal_load(
            reinterpret_cast<const u32x4*>(wrow + (c < nchunks ? c : 0) * 64));
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = chunk_of(p0, u);
      if (c < nchunks) {
        u32x4 xa[4];
        if (STAGED) {
          const u32x4* xp = reinterpret_cast<const u32x4*>(xrec + c * xrec_stride);
#pragma unroll
          for (int t = 0; t < 4; ++t) xa[t] = xp[t];
        } else {
          const u32x4* xp = reinterpret_cast<const u32x4*>(xrow + c * 128);
          u32x4 raw[4];
#pragma unroll
          for (int t = 0; t < 4; ++t) raw[t] = has_x ? xp[t] : zero4;
          permute_unit(raw[0], raw[1], xa[0], xa[1]);
          permute_unit(raw[2], raw[3], xa[2], xa[3]);
        }
        const float s = (float)slr[cpg_shift >= 0 ? (c >> cpg_shift) : (c * 128 / group_size)];
        // the accumulator starts at -(1032 * sum_lo x + 72 * sum_hi x) of the chunk: the x
        // operands against constant operands, four matrix instructions that do not depend on
        // the codes (summing the terms with vector instructions while x is staged was two thirds
        // of the staging pass)
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, xa[2 * h]), kn1032,
                                                       acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, xa[2 * h + 1]),
                                                       kn72, acc, 0, 0, 0);
        }
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const uint32_t w0 = wq[u][2 * h];
          const uint32_t w1 = wq[u][2 * h + 1];
          const uint32_t w0s = w0 >> 8, w1s = w1 >> 8;
          // (w & mask) ^ (magic | sign bit of the nibble): xor 8 and merge 0x6400 in one op
          u32x4 blo, bhi;
          blo[0] = (w0 & 0x000F000Fu) ^ 0x64086408u;
          blo[1] = (w0s & 0x000F000Fu) ^ 0x64086408u;
          blo[2] = (w1 & 0x000F000Fu) ^ 0x64086408u;
          blo[3] = (w1s & 0x000F000Fu) ^ 0x64086408u;
          bhi[0] = (w0 & 0x00F000F0u) ^ 0x54805480u;
          bhi[1] = (w0s & 0x00F000F0u) ^ 0x54805480u;
          bhi[2] = (w1 & 0x00F000F0u) ^ 0x54805480u;
          bhi[3] = (w1s & 0x00F000F0u) ^ 0x54805480u;
          const f16x8 a_lo = __builtin_bit_cast(f16x8, xa[2 * h]);
          const f16x8 a_hi = __builtin_bit_cast(f16x8, xa[2 * h + 1]);
          acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_lo, __builtin_bit_cast(f16x8, blo), acc,
                                                       0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_hi, __builtin_bit_cast(f16x8, bhi), acc,
                                                       0, 0, 0);
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) total[v] = __builtin_fmaf(acc[v], s, total[v]);
      }
    }
    if (pn < npairs) {
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) wq[u] = wq_next[u];
    }
  }
  // lane holds D[m = 4*kb + v][n = n0 + r]; only rows m < M travel through LDS
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const int m = 4 * kb + v;
    if (m < M) red[(wave * 16 + m) * 16 + r] = total[v];
  }
  __syncthreads();
  if (tid < M * 16) {
    float sum = 0.f;
#pragma unroll
    for (int wv = 0; wv < NWAVES; ++wv) sum += red[wv * 256 + tid];
    const int m = tid >> 4;
    const int n = n0 + (tid & 15);
    if (n < N) {
      sum += (float)bias_at_end(bias_raw);
      out[(int64_t)m * N + n] = (f16)sum;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Row-balanced variant of the fast path.  The grid is a whole number of blocks per CU and every
// block owns `rows_per_block` CONSECUTIVE weight rows (any count up to 16 * kW4pMaxTiles), which
// it walks as 16-row tiles with a partial last tile: all blocks stream the same number of bytes
// whatever n is (11008 rows = 43 per block on 256 CUs, where 16-row blocks would leave a third of
// the CUs a tile short), and x is permuted into LDS once per block, not once per 16 rows, which
// is what makes m > 1 affordable (the staged x is m*k*2 bytes per block).  The 16 waves take the
// (tile, chunk-pair) items of the block round-robin and keep one item in flight beyond the one
// they work on; partial sums go to LDS per (tile, wave) and are folded after a single barrier.
// Arithmetic is that of gemv_w4s_f16.
// ---------------------------------------------------------------------------------------------
constexpr int kW4pMaxTiles = 4;

// EXACT = false: the unrounded arithmetic above (int8 container, symmetric).
// EXACT = true : w~ = T(T(code) * s) + z formed with packed fp16 multiply and add exactly as the
//   reference does, for either container and any zero mode.  It is needed wherever a zero term
//   is involved: w~ is then a small difference of two values of magnitude ~7s, the reference's
//   three roundings are relative to those, and leaving them out moves the result by ~1e-3
//   relative to the dequantize->matmul composition (measured 6e-4 on uniform codes, more on
//   bell-shaped ones).  x is staged in the k-order of unpack4_pairs, one MFMA per code word.
// GLU mode: the block also owns the SAME rows of a second weight (the gate), as further tiles,
// and its last step forms y = T(hidden * T(act(gate))) from the two rounded sums
// (oneflow/user/kernels/fused_glu_kernel.cu:303-347); both sums are stored as well.
struct GluArgs {
  const uint8_t* w2;
  const f16* scale2;
  const f16* zero2;
  const f16* bias2;
  f16* out2;
  f16* y;
  int act;  // 0 none, 1 sigmoid, 2 relu, 3 gelu, 4 fast_gelu, 5 silu
};

// fp32 forms of oneflow/core/ep/common/primitive/unary_functor.h:146-170,477-484 and
// oneflow/core/ep/cuda/primitive/unary_functor.cuh:31-58
__device__ __forceinline__ float glu_activation(float v, int act) {
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

// TILED: w is the tile-major copy ofq_groupwise_repack writes (see w4p_tiled_bytes): the 64-byte
// chunk c of the 16 rows of the block's tile t is one contiguous KB in the order the lanes take
// it, [k-slot 0..3][row 0..15][16 bytes], at ((block * tiles_per_block + t) * nchunks + c) * 1024.
// A request of a wave is then 1 KB of consecutive bytes instead of 16 pieces of 64.
// PH > 1: m * k is more than LDS holds at once (8 rows of 11008): the chunk pairs of a row are
// walked in PH parts, each with its own staging of x; the x of the next part is requested while
// the current one is worked on, and the sums of a (tile, wave) add up in `red`.
template<int NWAVES, int kW4pDepth = 2, bool EXACT = false, bool SIGNED = true,
         int ZMODE = kZeroNone, bool GLU = false, bool TILED = false, int PH = 1>
__device__ __forceinline__ void
gemv_w4p_body(int block, const f16* __restrict__ x, const uint8_t* __restrict__ w,
              const f16* __restrict__ scale, const f16* __restrict__ zero,
              const f16* __restrict__ bias, f16* __restrict__ out, int M, int N, int K,
              int group_size, int cpg_shift, int rows_per_block, GluArgs glu = GluArgs()) {
  static_assert(EXACT || (SIGNED && ZMODE == kZeroNone), "the unrounded path has no zero term");
  static_assert(!(GLU && TILED), "the tile-major layout serves the plain linear only");
  static_assert(PH >= 1 && PH <= 4, "one to four stagings of x");
  constexpr int NMAT = GLU ? 2 : 1;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  constexpr int NT = NWAVES * 64;
  const int nchunks = K >> 7;
  const int npairs_all = (nchunks + 1) >> 1;
  // the phase being worked on: its chunk pairs [., + npairs), its chunks [cbeg, cbeg + ncs)
  const int pairs_per_phase = (npairs_all + PH - 1) / PH;
  int npairs = pairs_per_phase;
  int cbeg = 0;
  int ncs = PH > 1 && 2 * pairs_per_phase < nchunks ? 2 * pairs_per_phase : nchunks;
  uint32_t inv_chunks = row_of_inv(ncs);
  const int G = K / group_size;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15;
  const int kb = lane >> 4;
  const int row0 = block * rows_per_block;
  int rows_blk = N - row0;
  if (rows_blk > rows_per_block) rows_blk = rows_per_block;
  if (rows_blk <= 0) return;
  const int ntiles = (rows_blk + 15) >> 4;  // per weight
  const int nvt = NMAT * ntiles;            // tiles the block walks: the gate's follow the first's
  const bool has_x = r < M;
  // tile vt -> its weight (0 / 1), its first row within the block, its row of the scale tiles
  auto mat_of = [&](int vt) { return GLU && vt >= ntiles ? 1 : 0; };
  auto trow_of = [&](int vt) { return (GLU && vt >= ntiles ? vt - ntiles : vt) * 16; };
  auto srow_of = [&](int vt) { return (GLU && vt >= ntiles ? rows_per_block : 0) + trow_of(vt); };

  // LDS: [red NMAT*tiles_per_block*NWAVES*M*16 f32][scales NMAT*rows_per_block*G halves, padded to 16 B]
  //      [zeros, same size (asymmetric only)][64 zero bytes]
  //      [x records M*ncs*256 B, ncs = chunks of a phase]
  float* red = reinterpret_cast<float*>(smem);
  const int tiles_per_block = (rows_per_block + 15) >> 4;
  const int red_floats = NMAT * tiles_per_block * NWAVES * M * 16;  // <= kW4pMaxTiles tiles
  const int tile_bytes = (NMAT * rows_per_block * G * 2 + 15) & ~15;
  f16* sl = reinterpret_cast<f16*>(smem + (size_t)red_floats * 4);
  f16* zl = reinterpret_cast<f16*>(reinterpret_cast<uint8_t*>(sl) + tile_bytes);
  uint8_t* zrec = reinterpret_cast<uint8_t*>(sl) + (ZMODE == kZeroAsym ? 2 : 1) * tile_bytes;
  uint8_t* xs = zrec + 64;

  // ---- requests that feed LDS go out first ----------------------------------------------------
  int nunits = M * ncs * 8;  // 32-byte units of x of the phase, row by row
  u32x4 xu[kGemvMaxUnits][2];
  // unit u of a phase whose rows hold `cs` chunks from chunk `c0` on
  auto request_x = [&](int units, int cs, int c0, uint32_t inv) {
#pragma unroll
    for (int i = 0; i < kGemvMaxUnits; ++i) {
      if (wave * 64 + i * NT >= units) break;
      const int u = tid + i * NT;
      if (u < units) {
        const u32x4* src;
        if constexpr (PH == 1) {
          src = reinterpret_cast<const u32x4*>(x + (int64_t)u * 16);
        } else {
          const int m = row_of(u >> 3, inv);
          const int cl = (u >> 3) - m * cs;
          src = reinterpret_cast<const u32x4*>(x + ((int64_t)(m * nchunks + c0 + cl) * 8 + (u & 7)) * 16);
        }
        xu[i][0] = src[0];
        xu[i][1] = src[1];
      }
    }
  };
  request_x(nunits, ncs, cbeg, inv_chunks);
  // the scales of the block's rows are one contiguous piece
  const int tile_halves = rows_blk * G;
  const f16* stile = scale + (int64_t)row0 * G;
  const bool s_aligned = ((reinterpret_cast<uintptr_t>(stile)) & 15u) == 0;
  const f16* ztile = ZMODE == kZeroAsym ? zero + (int64_t)row0 * G : stile;  // same alignment
  u32x4 sreg, zreg;
  const int se = tid * 8;
  const bool s_vec = s_aligned && se + 8 <= tile_halves;
  if (s_vec) {
    sreg = *reinterpret_cast<const u32x4*>(stile + se);
    if (ZMODE == kZeroAsym) zreg = *reinterpret_cast<const u32x4*>(ztile + se);
  }
  // the gate's scales (GLU): same rows of the second weight, hence the same alignment
  const f16* stile2 = GLU ? glu.scale2 + (int64_t)row0 * G : stile;
  const f16* ztile2 = GLU && ZMODE == kZeroAsym ? glu.zero2 + (int64_t)row0 * G : stile2;
  const bool s_aligned2 = ((reinterpret_cast<uintptr_t>(stile2)) & 15u) == 0;
  const bool s_vec2 = GLU && s_aligned2 && se + 8 <= tile_halves;
  u32x4 sreg2, zreg2;
  if (GLU && s_vec2) {
    sreg2 = *reinterpret_cast<const u32x4*>(stile2 + se);
    if (ZMODE == kZeroAsym) zreg2 = *reinterpret_cast<const u32x4*>(ztile2 + se);
  }
  // bias of the output this thread folds at the end: tid = (tile * M + m) * 16 + n
  // (kept as raw bits: widening it here would wait for every load issued so far)
  uint16_t bias_raw = 0, bias_raw2 = 0;
  {
    const int t = tid / (M * 16);
    const int n = row0 + t * 16 + (tid & 15);
    if (bias != nullptr && t < ntiles && (t * 16 + (tid & 15)) < rows_blk) {
      bias_raw = reinterpret_cast<const uint16_t*>(bias)[n];
    }
    if (GLU && glu.bias2 != nullptr && t < ntiles && (t * 16 + (tid & 15)) < rows_blk) {
      bias_raw2 = reinterpret_cast<const uint16_t*>(glu.bias2)[n];
    }
  }

  // ---- the wave's items: j = wave, wave + NWAVES, ... over ntiles * npairs; the first
  // kW4pDepth of them are requested now, before anything is waited for (for the usual shapes
  // that is all of them: the block's whole share of the weights is in flight at once)
  const uint8_t* wbase = w + (int64_t)row0 * (K >> 1) + kb * 16;
  const uint8_t* wbase2 = GLU ? glu.w2 + (int64_t)row0 * (K >> 1) + kb * 16 : wbase;
  // Straight-line on purpose: a load under a branch (even a uniform one) makes the compiler
  // wait for everything in flight at the first LDS fill.  A slot without an item (live = false)
  // reads one and the same 16 bytes in every lane, a single cached request; lanes past the
  // block's rows re-read its first row (their outputs are never stored).
  auto issue = [&](int tile, int pair, u32x4 (&dst)[2], bool live) {
    if constexpr (TILED) {
      const uint8_t* tbase = w + ((int64_t)block * tiles_per_block + tile) * nchunks * 1024
                             + lane * 16;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int c = cbeg + 2 * pair + u;
        const uint8_t* q = tbase + (int64_t)(c < nchunks ? c : 0) * 1024;
        dst[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(live ? q : w));
      }
      return;
    }
    const int row_l = trow_of(tile) + r;
    const bool ok = row_l < rows_blk;
    const uint8_t* p = (mat_of(tile) ? wbase2 : wbase) + (int64_t)(ok ? row_l : 0) * (K >> 1);
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c = cbeg + 2 * pair + u;
      const uint8_t* q = p + (c < nchunks ? c : 0) * 64;
      dst[u] = __builtin_nontemporal_load(
          reinterpret_cast<const u32x4*>(live ? q : w + (int64_t)row0 * (K >> 1)));
    }
  };
  auto advance = [&](int& tile, int& pair, int by) {
    pair += by;
    while (pair >= npairs) {
      pair -= npairs;
      ++tile;
    }
  };
  int it_tile[kW4pDepth], it_pair[kW4pDepth];
  u32x4 wq[kW4pDepth][2];
  auto first_items = [&]() {
#pragma unroll
    for (int d = 0; d < kW4pDepth; ++d) {
      it_tile[d] = 0;
      it_pair[d] = wave + d * NWAVES;
      advance(it_tile[d], it_pair[d], 0);
      // unconditional, so that the wait counts stay exact: a slot without an item reads one and
      // the same 16 bytes in every lane (a single cached request)
      {
        const bool live = it_tile[d] < nvt;
        issue(live ? it_tile[d] : 0, live ? it_pair[d] : 0, wq[d], live);
      }
    }
  };
  first_items();

  // ---- fill LDS -------------------------------------------------------------------------------
  for (int e = tid; e < red_floats / 4; e += NT) reinterpret_cast<f32x4*>(red)[e] = f32x4{0.f, 0.f, 0.f, 0.f};
  if (s_vec) {
    *reinterpret_cast<u32x4*>(sl + se) = sreg;
    if (ZMODE == kZeroAsym) *reinterpret_cast<u32x4*>(zl + se) = zreg;
  } else if (se < tile_halves && s_aligned) {
    for (int j = se; j < tile_halves && j < se + 8; ++j) {
      sl[j] = stile[j];
      if (ZMODE == kZeroAsym) zl[j] = ztile[j];
    }
  }
  for (int e = (s_aligned ? NT * 8 : 0) + tid; e < tile_halves; e += NT) {
    sl[e] = stile[e];
    if (ZMODE == kZeroAsym) zl[e] = ztile[e];
  }
  if (GLU) {
    f16* sl2 = sl + rows_per_block * G;
    f16* zl2 = zl + rows_per_block * G;
    // (rows_per_block * G halves may leave sl2 off a 16-byte boundary: vector stores only
    // when it is on one)
    const bool lds_vec = ((rows_per_block * G) & 7) == 0;
    if (s_vec2 && lds_vec) {
      *reinterpret_cast<u32x4*>(sl2 + se) = sreg2;
      if (ZMODE == kZeroAsym) *reinterpret_cast<u32x4*>(zl2 + se) = zreg2;
    } else if (s_vec2) {
      const f16x8 sv = __builtin_bit_cast(f16x8, sreg2);
#pragma unroll
      for (int j = 0; j < 8; ++j) sl2[se + j] = sv[j];
      if (ZMODE == kZeroAsym) {
        const f16x8 zv = __builtin_bit_cast(f16x8, zreg2);
#pragma unroll
        for (int j = 0; j < 8; ++j) zl2[se + j] = zv[j];
      }
    } else if (se < tile_halves && s_aligned2) {
      for (int j = se; j < tile_halves && j < se + 8; ++j) {
        sl2[j] = stile2[j];
        if (ZMODE == kZeroAsym) zl2[j] = ztile2[j];
      }
    }
    for (int e = (s_aligned2 ? NT * 8 : 0) + tid; e < tile_halves; e += NT) {
      sl2[e] = stile2[e];
      if (ZMODE == kZeroAsym) zl2[e] = ztile2[e];
    }
  }
  if (tid < 16) reinterpret_cast<uint32_t*>(zrec)[tid] = 0u;
  // x of the phase (held in xu) -> records in LDS
  auto stage_x = [&]() {
#pragma unroll
    for (int i = 0; i < kGemvMaxUnits; ++i) {
      if (wave * 64 + i * NT >= nunits) break;
      const int u = tid + i * NT;
      if (EXACT) {
        // one record per code word: x in the pair order of unpack4_pairs
        if (u < nunits) {
          // rows of x are skewed by 16 bytes each: the lanes of different m that read the same
          // chunk then hit different LDS bank groups (their records are a multiple of 256 B apart)
          u32x4* dst = reinterpret_cast<u32x4*>(xs + (size_t)u * 32
                                                + row_of(u >> 3, inv_chunks) * 16);
          dst[0] = permute_x4(xu[i][0]);
          dst[1] = permute_x4(xu[i][1]);
        }
        continue;
      }
      if (u < nunits) {
        u32x4 lo, hi;
        permute_unit(xu[i][0], xu[i][1], lo, hi);
        u32x4* dst = reinterpret_cast<u32x4*>(xs + (size_t)u * 32
                                              + row_of(u >> 3, inv_chunks) * 16);
        dst[0] = lo;
        dst[1] = hi;
      }
      // (the correction terms are not summed here: sixteen conversions and additions per unit
      // were two thirds of this pass; the waves get them from the matrix core instead, see
      // process())
    }
  };
  stage_x();
  // chunks of phase ph (none when the row has fewer pairs than phases)
  auto phase_chunks = [&](int ph) {
    const int c0 = 2 * pairs_per_phase * ph;
    int cs = nchunks - c0;
    if (cs > 2 * pairs_per_phase) cs = 2 * pairs_per_phase;
    return cs > 0 ? cs : 0;
  };
  if constexpr (PH > 1) {
    // the next part's x goes out now; it is staged when this part has been walked
    const int cs = phase_chunks(1);
    request_x(M * cs * 8, cs, 2 * pairs_per_phase, row_of_inv(cs > 0 ? cs : 1));
  }
  __syncthreads();

  const uint8_t* xrec = has_x ? xs + (size_t)r * (ncs * 256 + 16) + kb * 64 : zrec;
  const int xrec_stride = has_x ? 256 : 0;
  bool add_to_red = false;  // later phases: the (tile, wave) slots already hold earlier sums
  const f16 c_lo = (f16)(-1032.0f), c_hi = (f16)(-72.0f);
  const f16x8 kn1032 = {c_lo, c_lo, c_lo, c_lo, c_lo, c_lo, c_lo, c_lo};
  const f16x8 kn72 = {c_hi, c_hi, c_hi, c_hi, c_hi, c_hi, c_hi, c_hi};
  f32x4 cneg[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
  int cneg_chunk[2] = {-1, -1};  // chunk (within the phase) whose correction terms cneg holds
  f32x4 total = {0.f, 0.f, 0.f, 0.f};
  f32x4 total1 = {0.f, 0.f, 0.f, 0.f};  // second accumulator of the exact path
  auto flush = [&](int t) {
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int m = 4 * kb + v;
      if (m < M) {
        float* slot = red + ((t * NWAVES + wave) * M + m) * 16 + r;
        const float sum = total[v] + total1[v];
        *slot = PH > 1 && add_to_red ? *slot + sum : sum;
      }
    }
    total1 = f32x4{0.f, 0.f, 0.f, 0.f};
  };

  // one item = the chunk pair `pair` of tile `tile`, codes in slot d
  auto process = [&](int d, int tile, int pair) {
    const f16* slr = sl + (srow_of(tile) + r) * G;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int cl = 2 * pair + u;  // chunk within the phase: the index of its x record
      const int c = cbeg + cl;
      if (c < nchunks) {
        const u32x4* xp = reinterpret_cast<const u32x4*>(xrec + cl * xrec_stride);
        u32x4 xa[4];
        if (!EXACT) {
          // only the lanes of rows of x that exist read: the other lanes' operands feed output
          // rows that are never stored, so whatever their registers hold will do
          if (has_x) {
#pragma unroll
            for (int t = 0; t < 4; ++t) xa[t] = xp[t];
          }
        } else {
#pragma unroll
          for (int t = 0; t < 4; ++t) xa[t] = xp[t];
        }
        const int grp = cpg_shift >= 0 ? (c >> cpg_shift) : (c * 128 / group_size);
        if (EXACT) {
          const f16 sh = slr[grp];
          f16 zh = (f16)0.0f;
          if (ZMODE == kZeroAsym) zh = zl[(srow_of(tile) + r) * G + grp];
          if (ZMODE == kZeroSymU) zh = (f16)(-7.0f) * sh;
          const f16x2 s2 = {sh, sh};
          const f16x2 z2 = {zh, zh};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            f16x2 p[4];
            unpack4_pairs<SIGNED>(wq[d][u][j], p);
            u32x4 bop;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              f16x2 v = p[e] * s2;
              if (ZMODE != kZeroNone) v = v + z2;
              bop[e] = as_u32(v);
            }
            // two accumulators: consecutive MFMAs do not wait for each other
            if (j & 1) {
              total1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                  __builtin_bit_cast(f16x8, xa[j]), __builtin_bit_cast(f16x8, bop), total1, 0, 0, 0);
            } else {
              total = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                  __builtin_bit_cast(f16x8, xa[j]), __builtin_bit_cast(f16x8, bop), total, 0, 0, 0);
            }
          }
          continue;
        }
        const float s = (float)slr[grp];
        // -(1032 * sum_lo x + 72 * sum_hi x) of the chunk for the lane's rows of x: the x operands
        // against constant operands, four matrix instructions that depend on LDS only and so
        // issue while the codes are still on their way.  Kept from one tile of the block to the
        // next: the tiles a wave walks mostly share their chunk pair.
        if (cl != cneg_chunk[u]) {
          f32x4 c0 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            c0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, xa[2 * h]), kn1032,
                                                        c0, 0, 0, 0);
            c0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, xa[2 * h + 1]),
                                                        kn72, c0, 0, 0, 0);
          }
          cneg[u] = c0;
          cneg_chunk[u] = cl;
        }
        f32x4 acc = cneg[u];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const uint32_t w0 = wq[d][u][2 * h];
          const uint32_t w1 = wq[d][u][2 * h + 1];
          const uint32_t w0s = w0 >> 8, w1s = w1 >> 8;
          u32x4 blo, bhi;
          blo[0] = (w0 & 0x000F000Fu) ^ 0x64086408u;
          blo[1] = (w0s & 0x000F000Fu) ^ 0x64086408u;
          blo[2] = (w1 & 0x000F000Fu) ^ 0x64086408u;
          blo[3] = (w1s & 0x000F000Fu) ^ 0x64086408u;
          bhi[0] = (w0 & 0x00F000F0u) ^ 0x54805480u;
          bhi[1] = (w0s & 0x00F000F0u) ^ 0x54805480u;
          bhi[2] = (w1 & 0x00F000F0u) ^ 0x54805480u;
          bhi[3] = (w1s & 0x00F000F0u) ^ 0x54805480u;
          acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, xa[2 * h]),
                                                       __builtin_bit_cast(f16x8, blo), acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, xa[2 * h + 1]),
                                                       __builtin_bit_cast(f16x8, bhi), acc, 0, 0, 0);
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) total[v] = __builtin_fmaf(acc[v], s, total[v]);
      }
    }
  };
  auto next_or_flush = [&](int d, int tile) {
    if (it_tile[(d + 1) % kW4pDepth] != tile) {
      flush(tile);
      total = f32x4{0.f, 0.f, 0.f, 0.f};
    }
  };
  auto walk = [&]() {
    // items of this wave: wave, wave + NWAVES, ... < nitems
    const int nitems = nvt * npairs;
    int left = nitems > wave ? (nitems - wave + NWAVES - 1) / NWAVES : 0;
    // steady state: every slot is consumed and refilled unconditionally, so the compiler's wait
    // before each slot is exact (the 2 * (kW4pDepth - 1) younger loads stay in flight)
    while (left >= 2 * kW4pDepth) {
#pragma unroll
      for (int d = 0; d < kW4pDepth; ++d) {
        const int tile = it_tile[d], pair = it_pair[d];
        process(d, tile, pair);
        advance(it_tile[d], it_pair[d], kW4pDepth * NWAVES);
        issue(it_tile[d], it_pair[d], wq[d], true);
        next_or_flush(d, tile);
      }
      left -= kW4pDepth;
    }
    // tail: fewer than 2 * kW4pDepth items are left; at most kW4pDepth - 1 refills
#pragma unroll
    for (int d = 0; d < kW4pDepth; ++d) {
      const int tile = it_tile[d], pair = it_pair[d];
      if (d < left) {
        process(d, tile, pair);
        advance(it_tile[d], it_pair[d], kW4pDepth * NWAVES);
        if (d + kW4pDepth < left) issue(it_tile[d], it_pair[d], wq[d], true);
        next_or_flush(d, tile);
      }
    }
#pragma unroll
    for (int d = 0; d < kW4pDepth - 1; ++d) {
      const int tile = it_tile[d], pair = it_pair[d];
      if (d + kW4pDepth < left) {
        process(d, tile, pair);
        advance(it_tile[d], it_pair[d], kW4pDepth * NWAVES);
        next_or_flush(d, tile);
      }
    }
  };
  walk();
  if constexpr (PH > 1) {
    // the further parts of the chunk pairs: a part's first items are requested before the
    // barrier behind which the x records are replaced
#pragma unroll 1
    for (int ph = 1; ph < PH; ++ph) {
      cbeg = 2 * pairs_per_phase * ph;
      ncs = phase_chunks(ph);
      if (ncs <= 0) break;  // uniform
      npairs = (ncs + 1) >> 1;
      inv_chunks = row_of_inv(ncs);
      nunits = M * ncs * 8;
      add_to_red = true;
      cneg_chunk[0] = cneg_chunk[1] = -1;  // the chunk indices start over with other x
      total = f32x4{0.f, 0.f, 0.f, 0.f};
      first_items();
      __syncthreads();  // every wave has read its last x record and correction of the part before
      stage_x();
      if (ph + 1 < PH) {
        const int cs = phase_chunks(ph + 1);
        request_x(M * cs * 8, cs, 2 * pairs_per_phase * (ph + 1), row_of_inv(cs > 0 ? cs : 1));
      }
      __syncthreads();
      xrec = has_x ? xs + (size_t)r * (ncs * 256 + 16) + kb * 64 : zrec;
      walk();
    }
  }
  __syncthreads();
  if (tid < ntiles * M * 16) {
    const int t = tid / (M * 16);
    const int rem = tid - t * (M * 16);  // m * 16 + n
    float sum = 0.f;
#pragma unroll
    for (int wv = 0; wv < NWAVES; ++wv) sum += red[(t * NWAVES + wv) * M * 16 + rem];
    const int m = rem >> 4;
    const int row_l = t * 16 + (rem & 15);
    if (GLU) {
      float sum2 = 0.f;
#pragma unroll
      for (int wv = 0; wv < NWAVES; ++wv) sum2 += red[((t + ntiles) * NWAVES + wv) * M * 16 + rem];
      if (row_l < rows_blk) {
        const int64_t o = (int64_t)m * N + row0 + row_l;
        const f16 hidden = (f16)(sum + (float)bias_at_end(bias_raw));
        const f16 gate = (f16)(sum2 + (float)bias_at_end(bias_raw2));
        out[o] = hidden;
        glu.out2[o] = gate;
        glu.y[o] = hidden * (f16)glu_activation((float)gate, glu.act);
      }
    } else if (row_l < rows_blk) {
      out[(int64_t)m * N + row0 + row_l] = (f16)(sum + (float)bias_at_end(bias_raw));
    }
  }
}

template<int NWAVES, int kW4pDepth = 2, bool EXACT = false, bool SIGNED = true,
         int ZMODE = kZeroNone, bool TILED = false, int PH = 1>
__global__ void __launch_bounds__(NWAVES * 64)
gemv_w4p_f16(const f16* __restrict__ x, const uint8_t* __restrict__ w,
             const f16* __restrict__ scale, const f16* __restrict__ zero,
             const f16* __restrict__ bias, f16* __restrict__ out, int M, int N, int K,
             int group_size, int cpg_shift, int rows_per_block) {
  gemv_w4p_body<NWAVES, kW4pDepth, EXACT, SIGNED, ZMODE, false, TILED, PH>(
      blockIdx.x, x, w, scale, zero, bias, out, M, N, K, group_size, cpg_shift, rows_per_block);
}

// Several problems of equal m, k and quantisation in one launch: the grid is the concatenation
// of the problems' blocks; a block finds its problem in the table.
constexpr int kGemvMaxProblems = 8;
struct GemvProblem {
  const void* x;
  const uint8_t* w;
  const void* scale;
  const void* zero;
  const void* bias;
  void* out;
  int N;
  int first_block;  // of the grid
};
struct GemvGroup {
  GemvProblem p[kGemvMaxProblems];
  int count;
};
// (every field is selected with a chain of scalar selects over the table entries: indexing the
// argument struct with a run-time value, or copying an entry as a whole, moves the table to
// scratch memory)
__device__ __forceinline__ GemvProblem select_problem(const GemvGroup& g, int block) {
  int i = 0;
#pragma unroll
  for (int j = 1; j < kGemvMaxProblems; ++j) {
    if (j < g.count && block >= g.p[j].first_block) i = j;
  }
  GemvProblem pr;
#define OFQ_SEL(field)                                   \
  pr.field = g.p[0].field;                               \
  _Pragma("unroll") for (int j = 1; j < kGemvMaxProblems; ++j) { \
    if (i == j) pr.field = g.p[j].field;                 \
  }
  OFQ_SEL(x)
  OFQ_SEL(w)
  OFQ_SEL(scale)
  OFQ_SEL(zero)
  OFQ_SEL(bias)
  OFQ_SEL(out)
  OFQ_SEL(N)
  OFQ_SEL(first_block)
#undef OFQ_SEL
  return pr;
}

template<int NWAVES, bool EXACT, bool SIGNED, int ZMODE, int PH = 1>
__global__ void __launch_bounds__(NWAVES * 64)
gemv_w4p_f16_grouped(GemvGroup g, int M, int K, int group_size, int cpg_shift,
                     int rows_per_block) {
  const GemvProblem pr = select_problem(g, (int)blockIdx.x);
  gemv_w4p_body<NWAVES, 1, EXACT, SIGNED, ZMODE, false, false, PH>(
      (int)blockIdx.x - pr.first_block, static_cast<const f16*>(pr.x), pr.w,
      static_cast<const f16*>(pr.scale), static_cast<const f16*>(pr.zero),
      static_cast<const f16*>(pr.bias), static_cast<f16*>(pr.out), M, pr.N, K, group_size,
      cpg_shift, rows_per_block);
}

// two weights of equal shape (hidden state, gate), every block the same rows of both
template<int NWAVES, bool EXACT, bool SIGNED, int ZMODE, int PH = 1>
__global__ void __launch_bounds__(NWAVES * 64)
gemv_w4p_f16_glu(const f16* __restrict__ x, const uint8_t* __restrict__ w,
                 const f16* __restrict__ scale, const f16* __restrict__ zero,
                 const f16* __restrict__ bias, f16* __restrict__ out, GluArgs glu, int M, int N,
                 int K, int group_size, int cpg_shift, int rows_per_block) {
  gemv_w4p_body<NWAVES, 1, EXACT, SIGNED, ZMODE, true, false, PH>(
      blockIdx.x, x, w, scale, zero, bias, out, M, N, K, group_size, cpg_shift, rows_per_block,
      glu);
}

// chunks of x a block holds at once: all of a row's, or (several stagings) the largest part of
// its chunk pairs
inline int gemv_w4p_phase_chunks(int K, int phases) {
  const int nchunks = K >> 7;
  const int per_phase = 2 * ((((nchunks + 1) >> 1) + phases - 1) / phases);
  return phases > 1 && per_phase < nchunks ? per_phase : nchunks;
}

inline size_t gemv_w4p_lds_bytes(int nwaves, int M, int K, int group_size, int rows_per_block,
                                 bool exact, bool asym, int nmat = 1, int phases = 1) {
  const int G = K / group_size;
  return (size_t)nmat * ((rows_per_block + 15) / 16) * nwaves * M * 16 * 4
         + (size_t)(asym ? 2 : 1) * ((nmat * rows_per_block * G * 2 + 15) & ~15) + 64
         + (size_t)M * (gemv_w4p_phase_chunks(K, phases) * 256 + 16);
}

// dynamic LDS bytes of gemv_w4s_f16
inline size_t gemv_w4s_lds_bytes(int nwaves, bool staged, int M, int K, int group_size) {
  const int G = K / group_size;
  return (size_t)nwaves * 64 * 16 + ((16 * G * 2 + 15) & ~15) + 64
         + (staged ? (size_t)M * (K * 2 + 16) : 0);
}

}  // namespace
}  // namespace ofq
