// Decode kernel for ONE row of x (m = 1) of fused_linear_with_groupwise_quantized_weight for
// every 16-bit element type, both code widths, both containers and both quantisation schemes,
// groups along K.
//
// The structure is the one of gemv_w4_m1.h, which serves the fp16 / 4-bit / signed / symmetric
// case: a WAVE owns whole weight rows, a lane reads 16 contiguous bytes of codes per KB of the
// row (1 KB per wave-level request), the k-reduction is a packed dot product per element pair in
// the lane plus one cross-lane sum per row, and x is staged once per block into LDS, lane-major.
// What differs is the arithmetic: the codes are expanded in NATURAL element order to
//   w~ = T(T(q) * s) + z  with the reference's roundings
//   (oneflow/user/kernels/groupwise_quantization_kernels.cu:73-117, :582-642)
// by dequant8_b4 / dequant16_b8, so a zero point, an unsigned container, 8-bit codes and bf16
// (whose rounded products have no shortcut) all take the same path, and x needs no permutation.
// The expansion is 3 to 6 VALU instructions per element (a wave64 instruction occupies its SIMD
// for four cycles): 4 to 8 us of issue per SIMD over a 45 M element weight, so this kernel is
// bound by the vector unit for bf16 with a zero point and close to it elsewhere; the launcher
// sends rows of more than 4096 elements to the MFMA kernels.
//
// A block owns rows_per_block consecutive rows, its wave w the rows w, w + NW, ..; the requests
// of a row (codes, scale, zero, bias) go out two rows ahead of its arithmetic.  With
// rows_per_block = NW this is one row per wave, every request of the block in flight at once.
#pragma once

#include "dequant_regs.h"
#include "gemv_rows.h"
#include "gemv_w4_m1.h"

namespace ofq {
namespace {

template<typename T>
__device__ __forceinline__ float dot2_t(uint32_t a, uint32_t b, float acc) {
  if constexpr (TT<T>::dtype == OFQ_BF16) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a),
                                           __builtin_bit_cast(bf16x2_t, b), acc, false);
  } else {
    return __builtin_amdgcn_fdot2(as_h2(a), as_h2(b), acc, false);
  }
}

// LDS: x as [KB h][piece t][lane l] 16-byte pieces
template<int BITS>
inline size_t gemv_m1_any_lds_bytes(int H) {
  return (size_t)H * (BITS == 4 ? 4096 : 2048);
}

// NW waves per block; H = KB of codes per row, rounded up (a lane owns bytes
// [h*1024 + lane*16, +16) of a row for h < H).
template<typename T, int BITS, bool SIGNED, int ZMODE, int NW, int H>
__global__ void __launch_bounds__(NW * 64)
gemv_m1_any(const uint16_t* __restrict__ x, const uint8_t* __restrict__ w,
            const uint16_t* __restrict__ scale, const uint16_t* __restrict__ zero,
            const uint16_t* __restrict__ bias, uint16_t* __restrict__ out, M1Shape sh) {
  typedef typename TT<T>::storage S;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  constexpr int NTH = NW * 64;
  constexpr int EPL = BITS == 4 ? 32 : 16;     // elements per lane and KB of codes
  constexpr int XP = EPL / 8;                  // 16-byte pieces of x per lane and KB
  constexpr int XU = (H * XP + NW - 1) / NW;   // pieces of x a thread stages
  constexpr bool kXInRegs = H * XP <= 8;       // x stays in registers across rows
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int K = sh.K;
  const int row_bytes = BITS == 4 ? K >> 1 : K;
  asm volatile("" ::"s"(out));
  const int row0 = blockIdx.x * sh.rows_per_block;
  int rows_blk = sh.N - row0;
  if (rows_blk > sh.rows_per_block) rows_blk = sh.rows_per_block;
  const int nr = rows_blk > wave ? (rows_blk - wave + NW - 1) / NW : 0;  // rows of this wave

  // ---- requests: x (feeds LDS, so it goes first), then two rows of the wave --------------------
  const int nunits = K >> 3;  // 16-byte pieces of x
  u32x4 xu[XU];
#pragma unroll
  for (int i = 0; i < XU; ++i) {
    if (wave * 64 + i * NTH >= nunits) break;  // wave-uniform
    int u = tid + i * NTH;
    u = u < nunits ? u : nunits - 1;
    xu[i] = reinterpret_cast<const u32x4*>(x)[u];
  }
  const uint8_t* wblk = w + (int64_t)row0 * row_bytes;
  const uint16_t* sblk = scale + (int64_t)row0 * sh.G;
  const uint16_t* zblk = ZMODE == kZeroAsym ? zero + (int64_t)row0 * sh.G : sblk;
  bool valid[H];
  uint32_t voff[H];
  int goff[H];
#pragma unroll
  for (int h = 0; h < H; ++h) {
    valid[h] = h * 1024 + lane * 16 < row_bytes;
    voff[h] = valid[h] ? (uint32_t)(h * 1024 + lane * 16) : 0u;
    goff[h] = valid[h] ? (h * 64 * EPL + lane * EPL) >> sh.gshift : 0;
  }
  u32x4 wq[2][H];
  uint16_t sc[2][H];
  uint16_t zr[2][H];
  uint16_t braw[2];
  // Every request is unconditional so that the wait counts stay exact: a slot past the wave's
  // last row reads one and the same 16 bytes in every lane (a single cached request).
  auto issue = [&](int i, int buf) {
    const bool live = i < nr;  // wave-uniform
    const int row_l = live ? wave + i * NW : 0;
    const uint8_t* rowp = wblk + (size_t)row_l * row_bytes;
    const uint16_t* srow = sblk + (size_t)row_l * sh.G;
    const uint16_t* zrow = zblk + (size_t)row_l * sh.G;
    // scales first: the arithmetic of the first KB can start when that KB has arrived, with
    // the rest of the row still in flight
#pragma unroll
    for (int h = 0; h < H; ++h) {
      sc[buf][h] = srow[live ? goff[h] : 0];
      if (ZMODE == kZeroAsym) zr[buf][h] = zrow[live ? goff[h] : 0];
    }
    braw[buf] = bias != nullptr ? bias[row0 + row_l] : (uint16_t)0;
#pragma unroll
    for (int h = 0; h < H; ++h) {
      wq[buf][h] = __builtin_nontemporal_load(
          reinterpret_cast<const u32x4*>(rowp + (live ? voff[h] : 0u)));
    }
  };
  issue(0, 0);

  // ---- x -> LDS: piece t of lane l of KB h at ((h*XP + t)*64 + l)*16 ---------------------------
#pragma unroll
  for (int i = 0; i < XU; ++i) {
    if (wave * 64 + i * NTH >= nunits) break;  // wave-uniform
    const int u = tid + i * NTH;
    const int c = u / XP;  // the lane-and-KB share of the row this piece belongs to
    const int h = c >> 6, l = c & 63, t = u % XP;
    if (u < nunits) {
      *reinterpret_cast<u32x4*>(smem + (size_t)(((h * XP + t) * 64 + l) * 16)) = xu[i];
    }
  }
  __syncthreads();
  issue(1, 1);  // behind the barrier: a smaller first burst streams a little better

  u32x4 xr[kXInRegs ? H : 1][XP];
  if (kXInRegs) {
#pragma unroll
    for (int h = 0; h < H; ++h) {
#pragma unroll
      for (int t = 0; t < XP; ++t) {
        xr[h][t] = *reinterpret_cast<const u32x4*>(smem + (size_t)(((h * XP + t) * 64 + lane) * 16));
      }
    }
  }
  auto finish = [&](int i, int buf) {
    float tot = 0.f;
#pragma unroll
    for (int h = 0; h < H; ++h) {
      u32x4 xa[XP];
#pragma unroll
      for (int t = 0; t < XP; ++t) {
        xa[t] = kXInRegs ? xr[kXInRegs ? h : 0][t]
                         : *reinterpret_cast<const u32x4*>(
                               smem + (size_t)(((h * XP + t) * 64 + lane) * 16));
      }
      const float s = raw16_at_end<T>(sc[buf][h]);
      float z = 0.f;
      if (ZMODE == kZeroAsym) z = raw16_at_end<T>(zr[buf][h]);
      if (ZMODE == kZeroSymU) z = TT<T>::round(-(float)((1 << (BITS - 1)) - 1) * s);
      float acc = 0.f;
      if constexpr (BITS == 4) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const u32x4 v = dequant8_b4<T, SIGNED, ZMODE>(wq[buf][h][t], s, z);
#pragma unroll
          for (int e = 0; e < 4; ++e) acc = dot2_t<T>(v[e], xa[t][e], acc);
        }
      } else {
        u32x4 v0, v1;
        dequant16_b8<T, SIGNED, ZMODE>(wq[buf][h], s, z, v0, v1);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc = dot2_t<T>(v0[e], xa[0][e], acc);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc = dot2_t<T>(v1[e], xa[1][e], acc);
      }
      tot += valid[h] ? acc : 0.f;
    }
    const float sum = wave_sum_m1(tot);
    if (lane == 0) {
      TT<T>::store(reinterpret_cast<S*>(out) + row0 + wave + i * NW,
                   sum + raw16_at_end<T>(braw[buf]));
    }
  };
  for (int i = 0; i < nr; i += 2) {
    finish(i, 0);
    issue(i + 2, 0);
    if (i + 1 < nr) finish(i + 1, 1);
    issue(i + 3, 1);
  }
}

}  // namespace
}  // namespace ofq
