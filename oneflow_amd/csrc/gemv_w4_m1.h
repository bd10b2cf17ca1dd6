// Decode kernel for ONE row of x (m = 1) of fused_linear_with_groupwise_quantized_weight:
// fp16, 4-bit symmetric codes in an int8 container, groups along K with 128 | group_size (a power
// of two times 128), K a multiple of 256.
//
// A decode linear on this chip is a one-shot kernel that ends one HBM round trip after it
// started, so what counts is what stands in front of the first request and behind the last byte.
// Measured on 4096 x 4096 (launch to launch, weights cold): the weights alone, requested 1 KB
// per instruction, take 2.7 us; requested as an MFMA operand layout wants them (adjacent lanes in
// different rows) 3.1 us; and the MFMA kernel 4.1 us, of which the cross-wave fold behind a
// barrier is 0.56 us, the per-lane scale gathers 0.2 us and the arithmetic itself next to
// nothing.  For one row of x the matrix core has nothing to offer either: 15 of its 16 rows are
// idle, and a packed dot product (v_dot2_f32_f16) reaches the same 32 useful MACs per clock.
//
// So here a WAVE owns whole weight rows:
//   - a lane reads 16 contiguous bytes, a wave-level request is 1 KB of one row: the cheapest
//     pattern for the address pipe and for DRAM;
//   - the k-reduction is 16 dot2 per 16 bytes of codes in the lane plus one cross-lane sum per row
//     (DPP), so there is no LDS fold, no second barrier, and a wave stores its row's output the
//     moment its own data has arrived;
//   - the scales of a row are 2 bytes per lane out of one or two cache lines, requested behind
//     the weights;
//   - x is permuted into the order the nibble masks deliver the codes ONCE per block, into LDS,
//     laid out lane-major, and every wave copies it to registers while the weights are in
//     flight.
// Arithmetic as in gemv_kernels.h: the half 0x6400|nibble is 1032+q (low nibbles), the half
// 0x5400|nibble<<4 is 72+q (high nibbles); the constant part per lane, 1032*sum_lo(x) + 72*sum_hi(x), is
// computed at staging and seeds the accumulator negated; products are exact in fp32, the group
// scale multiplies the lane's fp32 sum (w~ = q*s is not rounded to fp16).
#pragma once

#include "gemv_kernels.h"

namespace ofq {
namespace {

struct M1Shape {
  int N, K;
  int rows_per_block;
  int gshift;  // log2(group_size)
  int G;       // groups per row
  int gn;      // groups along N (GN kernels): rows per group, a multiple of rows_per_block
};

// LDS: [x operands H x 4 pieces x 64 lanes x 16 B] [corr H x 64 f32] [GN: power of two H x 64 f32]
inline size_t gemv_m1_lds_bytes(int H) { return (size_t)H * 4096 + (size_t)H * 512; }

template<int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
// sum over the 64 lanes, the same value in every lane's view of lanes 0, 16, 32, 48
__device__ __forceinline__ float wave_sum_m1(float v) {
  v += dpp_f32<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_f32<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_f32<0x141>(v);  // row_half_mirror
  v += dpp_f32<0x140>(v);  // row_mirror: every lane of a row of 16 holds the row's sum
  const float a = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
  const float b = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
  const float c = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
  const float d = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
  return (a + b) + (c + d);
}

// 16 bytes of codes (32 k) against the lane's x operands: xa[0]/xa[1] = low/high nibbles of words
// 0,1, xa[2]/xa[3] = of words 2,3 (the layout permute_unit writes)
__device__ __forceinline__ float m1_dot32(const u32x4 wq, const u32x4 (&xa)[4], float acc) {
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const uint32_t w0 = wq[2 * h];
    const uint32_t w1 = wq[2 * h + 1];
    const uint32_t w0s = w0 >> 8, w1s = w1 >> 8;
    uint32_t blo[4], bhi[4];
    blo[0] = (w0 & 0x000F000Fu) ^ 0x64086408u;
    blo[1] = (w0s & 0x000F000Fu) ^ 0x64086408u;
    blo[2] = (w1 & 0x000F000Fu) ^ 0x64086408u;
    blo[3] = (w1s & 0x000F000Fu) ^ 0x64086408u;
    bhi[0] = (w0 & 0x00F000F0u) ^ 0x54805480u;
    bhi[1] = (w0s & 0x00F000F0u) ^ 0x54805480u;
    bhi[2] = (w1 & 0x00F000F0u) ^ 0x54805480u;
    bhi[3] = (w1s & 0x00F000F0u) ^ 0x54805480u;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      acc = __builtin_amdgcn_fdot2(as_h2(blo[e]), as_h2(xa[2 * h][e]), acc, false);
      acc = __builtin_amdgcn_fdot2(as_h2(bhi[e]), as_h2(xa[2 * h + 1][e]), acc, false);
    }
  }
  return acc;
}

// The gate of a fused GLU: the same rows of a second weight of equal shape, owned by the same
// wave, which then forms y = T(hidden * T(act(gate))) itself
// (oneflow/user/kernels/fused_glu_kernel.cu:303-347); both linears are stored as well.
struct M1Glu {
  const uint8_t* w2;
  const f16* scale2;
  const f16* bias2;
  f16* out2;
  f16* y;
  int act;
};

// NW waves per block; RPW rows per wave (rows wave, wave + NW, ..); H = KB of codes per row,
// rounded up (a lane owns bytes [h*1024 + lane*16, +16) of a row for h < H); XU units of x per
// thread at staging; NM = 1, or 2 for the GLU (hidden and gate).
// GN: groups run along N (scale [N / gn, K], one value per k, shared by the gn rows of a group;
// a block's rows lie in one group).  The scale then meets x instead of the codes: the block
// stages x * s (one fp16 rounding per k, where the reference rounds q * s per element; a power of
// two per lane piece keeps the rounded value a normal half) and the rows need no scale of their
// own.
// D: KB of a row requested ahead of the arithmetic (D >= H: the whole row up front).  A CU
// keeps about 32 KB of requests in flight; a wave that asks for more than its share stands in the
// issue of its requests while its first KB has long arrived, and reaches the staging barrier late.
// With D = 3 of a long row the barrier is passed after 1 us instead of 2 to 4 (4096 x 11008), the
// arithmetic of a KB runs while the next ones arrive, and 16 waves per CU overlap better than two
// blocks of 8 (4096 x 11008: 6.2 -> 5.8 us, 4096 x 16384: 8.4 -> 7.3 us).
template<int NW, int RPW, int H, int XU, int NM, bool GN = false, int D = H>
__device__ __forceinline__ void
m1_body(int block, const f16* __restrict__ x, const uint8_t* __restrict__ w,
        const f16* __restrict__ scale, const f16* __restrict__ bias, f16* __restrict__ out, int N,
        const M1Shape& sh, const M1Glu& glu) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  constexpr int NTH = NW * 64;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int K = sh.K;
  const int row_bytes = K >> 1;
  const int row0 = block * sh.rows_per_block;
  int rows_blk = N - row0;
  if (rows_blk > sh.rows_per_block) rows_blk = sh.rows_per_block;

  // ---- requests: x (feeds LDS, so it goes first), bias, weights, scales -----------------------
  const int nunits = K >> 4;  // 32-byte units of x; XU per thread (K <= 16 * XU * NW * 64)
  const bool stage_wave = wave * 64 < nunits;  // wave-uniform
  u32x4 xu[XU][2];
  u32x4 su[GN ? XU : 1][2];
  if (stage_wave) {
#pragma unroll
    for (int i = 0; i < XU; ++i) {
      int u = tid + i * NTH;
      u = u < nunits ? u : nunits - 1;
      const u32x4* src = reinterpret_cast<const u32x4*>(x) + (size_t)u * 2;
      xu[i][0] = src[0];
      xu[i][1] = src[1];
      if (GN) {
        const u32x4* ssrc =
            reinterpret_cast<const u32x4*>(scale + (size_t)(row0 / sh.gn) * K) + (size_t)u * 2;
        su[GN ? i : 0][0] = ssrc[0];
        su[GN ? i : 0][1] = ssrc[1];
      }
    }
  }
  uint16_t bias_raw[NM][RPW];
#pragma unroll
  for (int q = 0; q < NM; ++q) {
    const f16* bq = q == 0 ? bias : glu.bias2;
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
      bias_raw[q][i] = 0;
      const int row_l = wave + i * NW;
      if (bq != nullptr) {
        bias_raw[q][i] = reinterpret_cast<const uint16_t*>(bq)[row0 + (row_l < rows_blk ? row_l : 0)];
      }
    }
  }
  u32x4 wq[NM][RPW][H];
  bool valid[H];
#pragma unroll
  for (int h = 0; h < H; ++h) valid[h] = h * 1024 + lane * 16 < row_bytes;
#pragma unroll
  for (int q = 0; q < NM; ++q) {
    const uint8_t* wblk = (q == 0 ? w : glu.w2) + (int64_t)row0 * row_bytes;
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
      const int row_l = wave + i * NW;
      const uint8_t* rowp = wblk + (size_t)(row_l < rows_blk ? row_l : 0) * row_bytes;
#pragma unroll
      for (int h = 0; h < (D < H ? D : H); ++h) {
        const uint32_t off = valid[h] ? (uint32_t)(h * 1024 + lane * 16) : 0u;
        wq[q][i][h] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(rowp + off));
      }
    }
  }
  f16 sc[NM][RPW][H];
#pragma unroll
  for (int q = 0; q < NM; ++q) {
    const f16* sblk = (q == 0 ? scale : glu.scale2) + (int64_t)row0 * sh.G;
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
      const int row_l = wave + i * NW;
      const f16* srow = sblk + (size_t)(row_l < rows_blk ? row_l : 0) * sh.G;
#pragma unroll
      for (int h = 0; h < H; ++h) {
        const int g = valid[h] ? (h * 2048 + lane * 32) >> sh.gshift : 0;
        sc[q][i][h] = GN ? (f16)1.0f : srow[g];
      }
    }
  }

  // ---- x -> LDS: piece t of lane l of KB h at ((h*4 + t)*64 + l)*16 ---------------------------
  float* corr_l = reinterpret_cast<float*>(smem + (size_t)H * 4096);
#pragma unroll
  for (int i = 0; i < XU; ++i) {
    if (wave * 64 + i * NTH >= nunits) break;  // wave-uniform
    const int u = tid + i * NTH;
    const bool ok = u < nunits;
    float unscale = 1.f;
    if (GN) {
      // x * s is exact in fp32.  The 32 products of a lane's piece (this unit and its
      // neighbour's) are brought to a common power of two that puts the largest in [2^12, 2^13)
      // before the one rounding to fp16, so that no product of ordinary size lands among the
      // subnormal halves whatever the magnitudes of x and s; the inverse power multiplies the
      // lane's fp32 sum.
      float v[2][8];
      float amax = 0.f;
#pragma unroll
      for (int p2 = 0; p2 < 2; ++p2) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          // (each word through a scalar of its own, see dequant8_b4_v)
          const uint32_t xw_u = xu[i][p2][e];
          const uint32_t sw_u = su[GN ? i : 0][p2][e];
          const f16x2 xw = as_h2(xw_u);
          const f16x2 sw = as_h2(sw_u);
          v[p2][2 * e] = (float)xw[0] * (float)sw[0];
          v[p2][2 * e + 1] = (float)xw[1] * (float)sw[1];
          amax = fmaxf(amax, fmaxf(fabsf(v[p2][2 * e]), fabsf(v[p2][2 * e + 1])));
        }
      }
      amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
      const int eb = (__builtin_bit_cast(int, amax) >> 23) & 0xFF;  // 0 (zero), or 79 .. 159
      const bool live = eb >= 64 && eb < 192;
      const float up = live ? __builtin_bit_cast(float, (266 - eb) << 23) : 1.f;    // 2^(12 - e)
      unscale = live ? __builtin_bit_cast(float, (eb - 12) << 23) : 1.f;            // 2^(e - 12)
#pragma unroll
      for (int p2 = 0; p2 < 2; ++p2) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const f16x2 r = {(f16)(v[p2][2 * e] * up), (f16)(v[p2][2 * e + 1] * up)};
          xu[i][p2][e] = as_u32(r);
        }
      }
    }
    u32x4 lo, hi;
    permute_unit(xu[i][0], xu[i][1], lo, hi);
    const int h = u >> 7, l = (u >> 1) & 63, p = u & 1;
    if (ok) {
      *reinterpret_cast<u32x4*>(smem + (size_t)(((h * 4 + 2 * p) * 64 + l) * 16)) = lo;
      *reinterpret_cast<u32x4*>(smem + (size_t)(((h * 4 + 2 * p + 1) * 64 + l) * 16)) = hi;
    }
    float cpart = ok ? unit_corr(lo, hi) : 0.f;
    cpart += __shfl_xor(cpart, 1, 64);
    if (ok && p == 0) {
      corr_l[h * 64 + l] = -cpart;
      if (GN) corr_l[(H + h) * 64 + l] = unscale;
    }
  }
  __syncthreads();

  // ---- per KB of the row: operands from LDS, then the rows of the wave -------------------------
  float tot[NM][RPW];
#pragma unroll
  for (int q = 0; q < NM; ++q) {
#pragma unroll
    for (int i = 0; i < RPW; ++i) tot[q][i] = 0.f;
  }
#pragma unroll
  for (int h = 0; h < H; ++h) {
    if (h + D < H) {
      // the KB D ahead, for every row of the wave
#pragma unroll
      for (int q = 0; q < NM; ++q) {
        const uint8_t* wblk = (q == 0 ? w : glu.w2) + (int64_t)row0 * row_bytes;
#pragma unroll
        for (int i = 0; i < RPW; ++i) {
          const int row_l = wave + i * NW;
          const uint8_t* rowp = wblk + (size_t)(row_l < rows_blk ? row_l : 0) * row_bytes;
          const uint32_t off = valid[h + D] ? (uint32_t)((h + D) * 1024 + lane * 16) : 0u;
          wq[q][i][h + D] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(rowp + off));
        }
      }
    }
    u32x4 xa[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      xa[t] = *reinterpret_cast<const u32x4*>(smem + (size_t)(((h * 4 + t) * 64 + lane) * 16));
    }
    const float cr = corr_l[h * 64 + lane];
#pragma unroll
    for (int q = 0; q < NM; ++q) {
#pragma unroll
      for (int i = 0; i < RPW; ++i) {
        const float acc = m1_dot32(wq[q][i][h], xa, cr);
        const float term = acc * (GN ? corr_l[(H + h) * 64 + lane] : (float)sc[q][i][h]);
        tot[q][i] += valid[h] ? term : 0.f;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < RPW; ++i) {
    const int row_l = wave + i * NW;
    const float sum = wave_sum_m1(tot[0][i]);
    if (NM == 1) {
      if (lane == 0 && row_l < rows_blk) {
        out[row0 + row_l] = (f16)(sum + (float)bias_at_end(bias_raw[0][i]));
      }
    } else {
      const float sum2 = wave_sum_m1(tot[NM - 1][i]);
      if (lane == 0 && row_l < rows_blk) {
        const f16 hidden = (f16)(sum + (float)bias_at_end(bias_raw[0][i]));
        const f16 gate = (f16)(sum2 + (float)bias_at_end(bias_raw[NM - 1][i]));
        out[row0 + row_l] = hidden;
        glu.out2[row0 + row_l] = gate;
        glu.y[row0 + row_l] = hidden * (f16)glu_activation((float)gate, glu.act);
      }
    }
  }
}

// The same for MANY rows per wave (n beyond what one resident round of one-row waves covers): a
// block owns rows_per_block consecutive rows, its wave w the rows w, w + NW, ..; x is staged once
// per block; the requests of a row go out two rows ahead of its arithmetic, so that a wave always
// has two rows (2 x H KB) in flight and the CU streams without the round trip a new block pays.
// Every request is unconditional so that the wait counts stay exact: a slot past the wave's last
// row reads one and the same 16 bytes in every lane (a single cached request).
template<int NW, int H, int XU>
__global__ void __launch_bounds__(NW * 64)
gemv_w4_m1_stream(const f16* __restrict__ x, const uint8_t* __restrict__ w,
                  const f16* __restrict__ scale, const f16* __restrict__ bias,
                  f16* __restrict__ out, M1Shape sh) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  constexpr int NTH = NW * 64;
  constexpr bool kXInRegs = H <= 2;  // x operands stay in registers across rows
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int K = sh.K;
  const int row_bytes = K >> 1;
  asm volatile("" ::"s"(out));
  const int row0 = blockIdx.x * sh.rows_per_block;
  int rows_blk = sh.N - row0;
  if (rows_blk > sh.rows_per_block) rows_blk = sh.rows_per_block;
  const int nr = rows_blk > wave ? (rows_blk - wave + NW - 1) / NW : 0;  // rows of this wave

  const int nunits = K >> 4;
  const bool stage_wave = wave * 64 < nunits;  // wave-uniform
  u32x4 xu[XU][2];
  if (stage_wave) {
#pragma unroll
    for (int i = 0; i < XU; ++i) {
      int u = tid + i * NTH;
      u = u < nunits ? u : nunits - 1;
      const u32x4* src = reinterpret_cast<const u32x4*>(x) + (size_t)u * 2;
      xu[i][0] = src[0];
      xu[i][1] = src[1];
    }
  }
  const uint8_t* wblk = w + (int64_t)row0 * row_bytes;
  const f16* sblk = scale + (int64_t)row0 * sh.G;
  bool valid[H];
  uint32_t voff[H];
  int goff[H];
#pragma unroll
  for (int h = 0; h < H; ++h) {
    valid[h] = h * 1024 + lane * 16 < row_bytes;
    voff[h] = valid[h] ? (uint32_t)(h * 1024 + lane * 16) : 0u;
    goff[h] = valid[h] ? (h * 2048 + lane * 32) >> sh.gshift : 0;
  }
  u32x4 wq[2][H];
  f16 sc[2][H];
  uint16_t braw[2];
  auto issue = [&](int i, int buf) {
    const bool live = i < nr;  // wave-uniform
    const int row_l = live ? wave + i * NW : 0;
    const uint8_t* rowp = wblk + (size_t)row_l * row_bytes;
    const f16* srow = sblk + (size_t)row_l * sh.G;
#pragma unroll
    for (int h = 0; h < H; ++h) {
      wq[buf][h] = __builtin_nontemporal_load(
          reinterpret_cast<const u32x4*>(rowp + (live ? voff[h] : 0u)));
    }
#pragma unroll
    for (int h = 0; h < H; ++h) sc[buf][h] = srow[live ? goff[h] : 0];
    braw[buf] = bias != nullptr ? reinterpret_cast<const uint16_t*>(bias)[row0 + row_l] : (uint16_t)0;
  };
  issue(0, 0);

  float* corr_l = reinterpret_cast<float*>(smem + (size_t)H * 4096);
#pragma unroll
  for (int i = 0; i < XU; ++i) {
    if (wave * 64 + i * NTH >= nunits) break;  // wave-uniform
    const int u = tid + i * NTH;
    const bool ok = u < nunits;
    u32x4 lo, hi;
    permute_unit(xu[i][0], xu[i][1], lo, hi);
    const int h = u >> 7, l = (u >> 1) & 63, p = u & 1;
    if (ok) {
      *reinterpret_cast<u32x4*>(smem + (size_t)(((h * 4 + 2 * p) * 64 + l) * 16)) = lo;
      *reinterpret_cast<u32x4*>(smem + (size_t)(((h * 4 + 2 * p + 1) * 64 + l) * 16)) = hi;
    }
    float cpart = ok ? unit_corr(lo, hi) : 0.f;
    cpart += __shfl_xor(cpart, 1, 64);
    if (ok && p == 0) corr_l[h * 64 + l] = -cpart;
  }
  __syncthreads();
  // the second row's requests go out behind the barrier: a smaller first burst streams a
  // little better than two rows per wave at once (8192 x 4096: 5.2 -> 5.0 us with the weights in
  // the memory-side cache, 11008 x 4096 from HBM: 6.6 -> 6.5 us)
  issue(1, 1);

  u32x4 xr[kXInRegs ? H : 1][4];
  float crr[kXInRegs ? H : 1];
  if (kXInRegs) {
#pragma unroll
    for (int h = 0; h < H; ++h) {
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        xr[h][t] = *reinterpret_cast<const u32x4*>(smem + (size_t)(((h * 4 + t) * 64 + lane) * 16));
      }
      crr[h] = corr_l[h * 64 + lane];
    }
  }
  auto finish = [&](int i, int buf) {
    float tot = 0.f;
#pragma unroll
    for (int h = 0; h < H; ++h) {
      float term;
      if (kXInRegs) {
        term = m1_dot32(wq[buf][h], xr[h], crr[h]) * (float)sc[buf][h];
      } else {
        u32x4 xa[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          xa[t] = *reinterpret_cast<const u32x4*>(smem + (size_t)(((h * 4 + t) * 64 + lane) * 16));
        }
        term = m1_dot32(wq[buf][h], xa, corr_l[h * 64 + lane]) * (float)sc[buf][h];
      }
      tot += valid[h] ? term : 0.f;
    }
    const float sum = wave_sum_m1(tot);
    if (lane == 0) out[row0 + wave + i * NW] = (f16)(sum + (float)bias_at_end(braw[buf]));
  };
  for (int i = 0; i < nr; i += 2) {
    finish(i, 0);
    issue(i + 2, 0);
    if (i + 1 < nr) finish(i + 1, 1);
    issue(i + 3, 1);
  }
}

// Many rows per wave for the fused GLU and for several problems in one launch (rows of at most
// 2 KB of codes): a block of the grid owns rows_per_block consecutive rows of ONE problem, stages
// that problem's x once, and each wave walks its rows wave, wave + NW, .. as one sequence of KB
// chunks with H chunks (one row) requested ahead of the arithmetic -- about 2 KB per wave and
// 32 KB per CU in flight, which is what a CU sustains; more only queues (two rows ahead, the
// plain streaming kernel's depth, was slower for these).  GLU: the sequence alternates between
// the row of the first weight and the same row of the gate weight, so a trip of the loop (two
// rows) is one (hidden, gate) pair and the wave that owns it forms y = hidden * act(gate).
// One resident round of blocks replaces the one-and-a-half rounds of one-row-per-wave blocks
// (2 x 11008 x 4096: 12.5 -> 9.7 us, three 4096 x 4096 problems: 7.8 -> 6.5 us).
template<int NW, int H, int XU, bool GLU>
__device__ __forceinline__ void
m1_walk_body(int block, const f16* __restrict__ x, const uint8_t* __restrict__ w,
             const f16* __restrict__ scale, const f16* __restrict__ bias, f16* __restrict__ out,
             int N, const M1Shape& sh, const M1Glu& glu) {
  static_assert(H == 1 || H == 2, "x operands stay in registers");
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  constexpr int NTH = NW * 64;
  constexpr int RING = 2 * H;  // two rows
  constexpr int D = H;         // one row ahead
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int K = sh.K;
  const int row_bytes = K >> 1;
  const int row0 = block * sh.rows_per_block;
  int rows_blk = N - row0;
  if (rows_blk > sh.rows_per_block) rows_blk = sh.rows_per_block;
  const int nr = rows_blk > wave ? (rows_blk - wave + NW - 1) / NW : 0;  // rows (GLU: pairs)
  const int nseq = GLU ? 2 * nr : nr;  // rows of the sequence
  const int nchunks = nseq * H;

  const int nunits = K >> 4;
  const bool stage_wave = wave * 64 < nunits;  // wave-uniform
  u32x4 xu[XU][2];
  if (stage_wave) {
#pragma unroll
    for (int i = 0; i < XU; ++i) {
      int u = tid + i * NTH;
      u = u < nunits ? u : nunits - 1;
      const u32x4* src = reinterpret_cast<const u32x4*>(x) + (size_t)u * 2;
      xu[i][0] = src[0];
      xu[i][1] = src[1];
    }
  }
  bool valid[H];
  uint32_t voff[H];
  int goff[H];
#pragma unroll
  for (int h = 0; h < H; ++h) {
    valid[h] = h * 1024 + lane * 16 < row_bytes;
    voff[h] = valid[h] ? (uint32_t)(h * 1024 + lane * 16) : 0u;
    goff[h] = valid[h] ? (h * 2048 + lane * 32) >> sh.gshift : 0;
  }
  u32x4 wq[RING];
  f16 sc[RING];
  uint16_t braw[2];
  // chunk c of the sequence: row c / H of the sequence (GLU: pair c / 2H, weight (c / H) & 1),
  // KB h of that row; slot c % RING.  Every request is unconditional so that the wait counts
  // stay exact: past the wave's last chunk all lanes read one and the same 16 bytes.
  auto issue = [&](int c, int slot, int h, int which) {
    const bool live = c < nchunks;  // wave-uniform
    const int i = live ? (GLU ? c / (2 * H) : c / H) : 0;
    const int row_l = live ? wave + i * NW : 0;
    const uint8_t* wb = (GLU && which) ? glu.w2 : w;
    const f16* sb = (GLU && which) ? glu.scale2 : scale;
    const f16* bb = (GLU && which) ? glu.bias2 : bias;
    const uint8_t* rowp = wb + (int64_t)(row0 + row_l) * row_bytes;
    wq[slot] = __builtin_nontemporal_load(
        reinterpret_cast<const u32x4*>(rowp + (live ? voff[h] : 0u)));
    sc[slot] = sb[(int64_t)(row0 + row_l) * sh.G + (live ? goff[h] : 0)];
    if (h == 0) {
      braw[(slot / H) & 1] =
          bb != nullptr ? reinterpret_cast<const uint16_t*>(bb)[row0 + row_l] : (uint16_t)0;
    }
  };
#pragma unroll
  for (int c = 0; c < D; ++c) issue(c, c % RING, c % H, (c / H) & 1);

  float* corr_l = reinterpret_cast<float*>(smem + (size_t)H * 4096);
#pragma unroll
  for (int i = 0; i < XU; ++i) {
    if (wave * 64 + i * NTH >= nunits) break;  // wave-uniform
    const int u = tid + i * NTH;
    const bool ok = u < nunits;
    u32x4 lo, hi;
    permute_unit(xu[i][0], xu[i][1], lo, hi);
    const int h = u >> 7, l = (u >> 1) & 63, p = u & 1;
    if (ok) {
      *reinterpret_cast<u32x4*>(smem + (size_t)(((h * 4 + 2 * p) * 64 + l) * 16)) = lo;
      *reinterpret_cast<u32x4*>(smem + (size_t)(((h * 4 + 2 * p + 1) * 64 + l) * 16)) = hi;
    }
    float cpart = ok ? unit_corr(lo, hi) : 0.f;
    cpart += __shfl_xor(cpart, 1, 64);
    if (ok && p == 0) corr_l[h * 64 + l] = -cpart;
  }
  __syncthreads();
  u32x4 xr[H][4];
  float crr[H];
#pragma unroll
  for (int h = 0; h < H; ++h) {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      xr[h][t] = *reinterpret_cast<const u32x4*>(smem + (size_t)(((h * 4 + t) * 64 + lane) * 16));
    }
    crr[h] = corr_l[h * 64 + lane];
  }
  for (int c0 = 0; c0 < nchunks; c0 += RING) {
    float tot = 0.f;
    float first = 0.f;  // the first row of the trip (GLU: hidden), bias added, rounded to T
#pragma unroll
    for (int j = 0; j < RING; ++j) {
      const int h = j % H;
      issue(c0 + j + D, (j + D) % RING, (j + D) % H, ((j + D) / H) & 1);
      const float term = m1_dot32(wq[j], xr[h], crr[h]) * (float)sc[j];
      tot += valid[h] ? term : 0.f;
      if (h == H - 1) {
        const float sum = wave_sum_m1(tot);
        const f16 v = (f16)(sum + (float)bias_at_end(braw[(j / H) & 1]));
        tot = 0.f;
        if (GLU) {
          const int row = row0 + wave + (c0 / RING) * NW;  // the pair of this trip
          if (j / H == 0) {
            first = (float)v;
            if (lane == 0) out[row] = v;
          } else if (lane == 0) {
            glu.out2[row] = v;
            glu.y[row] = (f16)first * (f16)glu_activation((float)v, glu.act);
          }
        } else {
          const int i = (c0 + j) / H;
          if (lane == 0 && i < nr) out[row0 + wave + i * NW] = v;
        }
      }
    }
  }
}

template<int NW, int H, int XU = 1>
__global__ void __launch_bounds__(NW * 64)
gemv_w4_m1_glu_walk(const f16* __restrict__ x, const uint8_t* __restrict__ w,
                    const f16* __restrict__ scale, const f16* __restrict__ bias,
                    f16* __restrict__ out, M1Glu glu, M1Shape sh) {
  m1_walk_body<NW, H, XU, true>(blockIdx.x, x, w, scale, bias, out, sh.N, sh, glu);
}

template<int NW, int H, int XU = 1>
__global__ void __launch_bounds__(NW * 64) gemv_w4_m1_grouped_walk(GemvGroup g, M1Shape sh) {
  const GemvProblem pr = select_problem(g, (int)blockIdx.x);
  m1_walk_body<NW, H, XU, false>((int)blockIdx.x - pr.first_block, static_cast<const f16*>(pr.x),
                                 pr.w, static_cast<const f16*>(pr.scale),
                                 static_cast<const f16*>(pr.bias), static_cast<f16*>(pr.out), pr.N,
                                 sh, M1Glu());
}

template<int NW, int RPW, int H, int XU = 1, int D = H>
__global__ void __launch_bounds__(NW * 64)
gemv_w4_m1(const f16* __restrict__ x, const uint8_t* __restrict__ w,
           const f16* __restrict__ scale, const f16* __restrict__ bias, f16* __restrict__ out,
           M1Shape sh) {
  asm volatile("" ::"s"(out));  // fetch the output pointer with the other arguments
  m1_body<NW, RPW, H, XU, 1, false, D>(blockIdx.x, x, w, scale, bias, out, sh.N, sh, M1Glu());
}

// groups along N: scale [N / sh.gn, K]
template<int NW, int H, int XU = 1>
__global__ void __launch_bounds__(NW * 64)
gemv_w4_m1_gn(const f16* __restrict__ x, const uint8_t* __restrict__ w,
              const f16* __restrict__ scale, const f16* __restrict__ bias, f16* __restrict__ out,
              M1Shape sh) {
  asm volatile("" ::"s"(out));
  m1_body<NW, 1, H, XU, 1, true>(blockIdx.x, x, w, scale, bias, out, sh.N, sh, M1Glu());
}

// hidden = x w~^T + b, gate = x v~^T + c, y = hidden * act(gate): one launch, one wave per row pair
template<int NW, int H, int XU = 1>
__global__ void __launch_bounds__(NW * 64)
gemv_w4_m1_glu(const f16* __restrict__ x, const uint8_t* __restrict__ w,
               const f16* __restrict__ scale, const f16* __restrict__ bias,
               f16* __restrict__ out, M1Glu glu, M1Shape sh) {
  m1_body<NW, 1, H, XU, 2>(blockIdx.x, x, w, scale, bias, out, sh.N, sh, glu);
}

// several problems of equal k in one launch: the grid is the concatenation of the problems'
// blocks, a block finds its problem in the table
template<int NW, int H, int XU = 1>
__global__ void __launch_bounds__(NW * 64) gemv_w4_m1_grouped(GemvGroup g, M1Shape sh) {
  const GemvProblem pr = select_problem(g, (int)blockIdx.x);
  m1_body<NW, 1, H, XU, 1>((int)blockIdx.x - pr.first_block, static_cast<const f16*>(pr.x), pr.w,
                           static_cast<const f16*>(pr.scale), static_cast<const f16*>(pr.bias),
                           static_cast<f16*>(pr.out), pr.N, sh, M1Glu());
}

}  // namespace
}  // namespace ofq
