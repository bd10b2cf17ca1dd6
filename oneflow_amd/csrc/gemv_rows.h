// Decode kernel of fused_linear_with_groupwise_quantized_weight for every 16-bit element type
// and both code widths, with x kept in its natural order.
//
// Same row split as gemv_w4p_f16 (a whole number of blocks per CU, each owning consecutive
// weight rows that it walks as 16-row tiles; the m <= 16 rows of x ride as the first operand of
// a 16x16x32 MFMA, so the weights stream from HBM once whatever m is), but the codes are
// expanded to T in natural element order by dequant8_b4 / dequant16_b8:
//   w~ = T(T(q) * s) + z  with the reference's roundings
//   (oneflow/user/kernels/groupwise_quantization_kernels.cu:73-117, :582-642),
// so bf16 (whose products have to be rounded in fp32 arithmetic: there is no packed bf16 math)
// and 8-bit codes get the same treatment as the fp16 4-bit case.  Groups may be as short as one
// lane's 16 bytes of codes (32 4-bit or 16 8-bit elements).
#pragma once

#include "dequant_regs.h"
#include "gemv_kernels.h"
#include "ofq_device.h"

namespace ofq {
namespace {

constexpr int kRowsMaxTiles = 4;   // 16-row tiles per block
constexpr int kRowsMaxUnits = 8;   // 16-byte pieces of x a thread may stage

template<typename T>
struct MfmaK32;
template<>
struct MfmaK32<f16> {
  static __device__ __forceinline__ f32x4 mma(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};
template<>
struct MfmaK32<bf16> {
  static __device__ __forceinline__ f32x4 mma(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};

// raw bits of a T -> float at the point of use (keeps the load's wait where the value is needed)
template<typename T>
__device__ __forceinline__ float raw16_at_end(uint16_t raw) {
  uint32_t v = raw;
  asm volatile("" : "+v"(v));
  if constexpr (TT<T>::dtype == OFQ_BF16) {
    return __builtin_bit_cast(float, v << 16);
  } else {
    return (float)__builtin_bit_cast(f16, (uint16_t)v);
  }
}

// STAGED: x is copied to LDS once per block (m * k small enough); otherwise every wave reads the
// x of its chunk pairs straight from global memory (x stays in L2: it is re-read by every block).
// Either way a wave takes chunk pairs p = wave, wave + NWAVES, ... and walks all tiles of the
// block for each, so x is fetched once per pair and the per-tile sums stay in registers.
template<typename T, int BITS, bool SIGNED, int ZMODE, int NWAVES, bool STAGED>
__device__ __forceinline__ void
gemv_rows_body(int block, const uint16_t* __restrict__ x, const uint8_t* __restrict__ w,
               const uint16_t* __restrict__ scale, const uint16_t* __restrict__ zero,
               const uint16_t* __restrict__ bias, uint16_t* __restrict__ out, int M, int N, int K,
               int group_size, int gs_shift, int rows_per_block) {
  typedef typename TT<T>::storage S;
  static_assert(sizeof(S) == 2, "16-bit element types");
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  constexpr int NT = NWAVES * 64;
  constexpr int CK = BITS == 4 ? 128 : 64;  // elements per chunk: 64 bytes of codes per row
  constexpr int LK = CK / 4;                // elements per lane and chunk
  constexpr int XV = LK / 8;                // 16-byte pieces of x per lane and chunk
  const int nchunks = K / CK;
  const int npairs = (nchunks + 1) >> 1;
  const int row_bytes = nchunks * 64;
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
  const int ntiles = (rows_blk + 15) >> 4;
  const bool has_x = r < M;

  // LDS: [scales rows_per_block*G, padded to 16 B][zeros, same size (asymmetric only)]
  //      [64 zero bytes][x: M rows of K*2+16 bytes (STAGED)]; the sums of the waves
  //      (tiles*NWAVES*M*16 f32) take the place of x once every wave has walked its pairs
  const int tile_bytes = (rows_per_block * G * 2 + 15) & ~15;
  uint16_t* sl = reinterpret_cast<uint16_t*>(smem);
  uint16_t* zl = reinterpret_cast<uint16_t*>(reinterpret_cast<uint8_t*>(sl) + tile_bytes);
  uint8_t* zrec = reinterpret_cast<uint8_t*>(sl) + (ZMODE == kZeroAsym ? 2 : 1) * tile_bytes;
  uint8_t* xs = zrec + 64;
  float* red = reinterpret_cast<float*>(xs);
  const int x_pitch = K * 2 + 16;  // rows skewed by 16 bytes: lanes of different m reading the
                                   // same k hit different LDS bank groups

  // ---- requests that feed LDS go out first ----------------------------------------------------
  const int upr = K >> 3;  // 16-byte pieces per row of x
  const int nunits = M * upr;
  u32x4 xu[kRowsMaxUnits];
  if (STAGED) {
#pragma unroll
    for (int i = 0; i < kRowsMaxUnits; ++i) {
      if (wave * 64 + i * NT >= nunits) break;
      const int u = tid + i * NT;
      if (u < nunits) xu[i] = *reinterpret_cast<const u32x4*>(x + (int64_t)u * 8);
    }
  }
  const int tile_halves = rows_blk * G;
  const uint16_t* stile = scale + (int64_t)row0 * G;
  const bool s_aligned = ((reinterpret_cast<uintptr_t>(stile)) & 15u) == 0;
  const uint16_t* ztile = ZMODE == kZeroAsym ? zero + (int64_t)row0 * G : stile;
  u32x4 sreg, zreg;
  const int se = tid * 8;
  const bool s_vec = s_aligned && se + 8 <= tile_halves;
  if (s_vec) {
    sreg = *reinterpret_cast<const u32x4*>(stile + se);
    if (ZMODE == kZeroAsym) zreg = *reinterpret_cast<const u32x4*>(ztile + se);
  }
  // bias of the first output this thread folds at the end: tid = (tile * M + m) * 16 + n
  uint16_t bias_raw = 0;
  {
    const int t = tid / (M * 16);
    const int row_l = t * 16 + (tid & 15);
    if (bias != nullptr && t < ntiles && row_l < rows_blk) bias_raw = bias[row0 + row_l];
  }

  // ---- codes of (tile, pair): one 16-byte load per lane and chunk ------------------------------
  const uint8_t* wbase = w + (int64_t)row0 * row_bytes + kb * 16;
  // Straight-line on purpose: a load under a branch makes the compiler wait for everything in
  // flight at the first LDS fill.  A slot without an item reads one and the same 16 bytes in
  // every lane; lanes past the block's rows re-read its first row (never stored).
  auto issue = [&](int tile, int pair, u32x4 (&dst)[2], bool live) {
    const int row_l = tile * 16 + r;
    const bool ok = row_l < rows_blk;
    const uint8_t* p = wbase + (int64_t)(ok ? row_l : 0) * row_bytes;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c = 2 * pair + u;
      const uint8_t* q = p + (c < nchunks ? c : 0) * 64;
      dst[u] = __builtin_nontemporal_load(
          reinterpret_cast<const u32x4*>(live ? q : w + (int64_t)row0 * row_bytes));
    }
  };
  int pair = wave;
  u32x4 wq[2];
  {
    const bool live = pair < npairs;
    issue(0, live ? pair : 0, wq, live);
  }

  // ---- fill LDS -------------------------------------------------------------------------------
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
  if (STAGED) {
    if (tid < 16) reinterpret_cast<uint32_t*>(zrec)[tid] = 0u;
    // piece u of x lies in row u / upr; rows advance by (NT / upr, NT % upr) per step
    const int qstep = NT / upr, rstep = NT - qstep * upr;
    int xrow = tid / upr, xrem = tid - xrow * upr;
#pragma unroll
    for (int i = 0; i < kRowsMaxUnits; ++i) {
      if (wave * 64 + i * NT >= nunits) break;
      if (tid + i * NT < nunits) {
        *reinterpret_cast<u32x4*>(xs + (size_t)xrow * x_pitch + xrem * 16) = xu[i];
      }
      xrow += qstep;
      xrem += rstep;
      if (xrem >= upr) {
        xrem -= upr;
        ++xrow;
      }
    }
  }
  __syncthreads();

  // this lane's 2 * LK bytes of x per chunk: row r, k-slot kb.  Lanes r >= M feed rows of the
  // product that are never stored: a zero record (STAGED) or row 0 again (same addresses as the
  // lanes of r = 0, no extra traffic).
  const uint8_t* xlane;
  int xstride = CK * 2;
  if (STAGED) {
    xlane = has_x ? xs + (size_t)r * x_pitch + kb * (LK * 2) : zrec;
    if (!has_x) xstride = 0;
  } else {
    xlane = reinterpret_cast<const uint8_t*>(x) + ((size_t)(has_x ? r : 0) * K + kb * LK) * 2;
  }
  f32x4 acc[kRowsMaxTiles][2];
#pragma unroll
  for (int t = 0; t < kRowsMaxTiles; ++t) {
    acc[t][0] = f32x4{0.f, 0.f, 0.f, 0.f};
    acc[t][1] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  while (pair < npairs) {
    u32x4 xa[2][XV];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c = 2 * pair + u;
      const u32x4* xp = reinterpret_cast<const u32x4*>(xlane + (size_t)(c < nchunks ? c : 0) * xstride);
#pragma unroll
      for (int j = 0; j < XV; ++j) xa[u][j] = xp[j];
    }
#pragma unroll
    for (int t = 0; t < kRowsMaxTiles; ++t) {
      if (t < ntiles) {
        const int srow = (t * 16 + r) * G;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int c = 2 * pair + u;
          if (c < nchunks) {
            const int k0 = c * CK + kb * LK;
            const int grp = gs_shift >= 0 ? (k0 >> gs_shift) : (k0 / group_size);
            const float s = TT<T>::load(reinterpret_cast<const S*>(sl) + srow + grp);
            float z = 0.f;
            if (ZMODE == kZeroAsym) z = TT<T>::load(reinterpret_cast<const S*>(zl) + srow + grp);
            if (ZMODE == kZeroSymU) z = TT<T>::round(-(float)((1 << (BITS - 1)) - 1) * s);
            if constexpr (BITS == 4) {
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                const u32x4 b = dequant8_b4<T, SIGNED, ZMODE>(wq[u][j], s, z);
                // two accumulators: consecutive MFMAs do not wait for each other
                acc[t][j & 1] = MfmaK32<T>::mma(xa[u][j], b, acc[t][j & 1]);
              }
            } else {
              u32x4 b0, b1;
              dequant16_b8<T, SIGNED, ZMODE>(wq[u], s, z, b0, b1);
              acc[t][0] = MfmaK32<T>::mma(xa[u][0], b0, acc[t][0]);
              acc[t][1] = MfmaK32<T>::mma(xa[u][1], b1, acc[t][1]);
            }
          }
        }
        // codes of the next item: the next tile of this pair, else tile 0 of the wave's next pair
        const bool last_t = t + 1 >= ntiles;
        const int np = last_t ? pair + NWAVES : pair;
        const bool live = np < npairs;
        issue(last_t ? 0 : t + 1, live ? np : 0, wq, live);
      }
    }
    pair += NWAVES;
  }
  // every wave writes its sums of every tile (zeros when it had no pair) where x was
  if (STAGED) __syncthreads();  // ... which every wave has finished reading
#pragma unroll
  for (int t = 0; t < kRowsMaxTiles; ++t) {
    if (t < ntiles) {
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int m = 4 * kb + v;
        if (m < M) red[((t * NWAVES + wave) * M + m) * 16 + r] = acc[t][0][v] + acc[t][1][v];
      }
    }
  }
  __syncthreads();
  const int nout = ntiles * M * 16;
  for (int o = tid; o < nout; o += NT) {
    const int t = o / (M * 16);
    const int rem = o - t * (M * 16);  // m * 16 + n
    float sum = 0.f;
#pragma unroll
    for (int wv = 0; wv < NWAVES; ++wv) sum += red[(t * NWAVES + wv) * M * 16 + rem];
    const int m = rem >> 4;
    const int row_l = t * 16 + (rem & 15);
    if (row_l < rows_blk) {
      float bv;
      if (o == tid) {
        bv = raw16_at_end<T>(bias_raw);
      } else {
        bv = bias != nullptr ? TT<T>::load(reinterpret_cast<const S*>(bias) + row0 + row_l) : 0.f;
      }
      TT<T>::store(reinterpret_cast<S*>(out) + (int64_t)m * N + row0 + row_l, sum + bv);
    }
  }
}

template<typename T, int BITS, bool SIGNED, int ZMODE, int NWAVES, bool STAGED>
__global__ void __launch_bounds__(NWAVES * 64)
gemv_rows(const uint16_t* __restrict__ x, const uint8_t* __restrict__ w,
          const uint16_t* __restrict__ scale, const uint16_t* __restrict__ zero,
          const uint16_t* __restrict__ bias, uint16_t* __restrict__ out, int M, int N, int K,
          int group_size, int gs_shift, int rows_per_block) {
  gemv_rows_body<T, BITS, SIGNED, ZMODE, NWAVES, STAGED>(blockIdx.x, x, w, scale, zero, bias, out,
                                                         M, N, K, group_size, gs_shift,
                                                         rows_per_block);
}

// Several linears of the same m, k and quantisation in one launch (q/k/v, gate/up ...): the grid
// is the concatenation of the problems' blocks, every problem cut into rows_per_block-row
// blocks; a block finds its problem in the table and runs the single-problem body on it.
template<typename T, int BITS, bool SIGNED, int ZMODE, int NWAVES, bool STAGED>
__global__ void __launch_bounds__(NWAVES * 64)
gemv_rows_grouped(GemvGroup g, int M, int K, int group_size, int gs_shift, int rows_per_block) {
  const GemvProblem pr = select_problem(g, (int)blockIdx.x);
  gemv_rows_body<T, BITS, SIGNED, ZMODE, NWAVES, STAGED>(
      (int)blockIdx.x - pr.first_block, static_cast<const uint16_t*>(pr.x), pr.w,
      static_cast<const uint16_t*>(pr.scale), static_cast<const uint16_t*>(pr.zero),
      static_cast<const uint16_t*>(pr.bias), static_cast<uint16_t*>(pr.out), M, pr.N, K,
      group_size, gs_shift, rows_per_block);
}

// ---------------------------------------------------------------------------------------------
// 16 < m <= 64: the same row split with MT = 2 or 4 sixteen-row tiles of x per MFMA group.  A
// weight tile is expanded once per chunk and meets all MT tiles of x, which come from L2 chunk
// by chunk (x is far too large for LDS here: m * k * 2 bytes per block); a wave walks chunks
// c = wave, wave + NWAVES, ... and, per chunk, every 16-row weight tile of the block, with the
// codes of the next (tile, chunk) requested before the current ones are used.  Sums stay in
// registers (kRowsMaxTiles * MT accumulators) and are folded through LDS one weight tile at a
// time.  No barrier inside the k loop, unlike the tiled GEMM, whose per-k-tile cost does not
// shrink with m.
// ---------------------------------------------------------------------------------------------
// XLDS: a lane's operand of x is 16 bytes out of a 64-byte run of one of 16 rows, so a
// wave-level request straight from global memory touches 64 cache lines for 1 KB of data and the
// vector cache's tag rate bounds the kernel (4096 x 11008 at 64 rows of x: 6 us per chunk and
// wave).  With XLDS a wave requests the chunk's MT * 16 rows x 2 CK bytes of x with neighbouring
// lanes on neighbouring bytes (8 cache lines per request), one chunk ahead, parks them in a
// buffer of its own in LDS (rows padded by 16 bytes) and reads its operands from there.  The
// buffers share their memory with the reduction area, which is used only after the k loop.
template<int BITS, int MT>
struct RowsMtX {
  static constexpr int CK = BITS == 4 ? 128 : 64;
  static constexpr int kRowBytes = CK * 2;           // of x per row and chunk
  static constexpr int kPitch = kRowBytes + 16;      // in LDS
  static constexpr int kLanesPerRow = kRowBytes / 16;
  static constexpr int kRowsPerReq = 64 / kLanesPerRow;
  static constexpr int kReqs = MT * 16 / kRowsPerReq;
  static constexpr int kWaveBytes = MT * 16 * kPitch;
};

template<typename T, int BITS, bool SIGNED, int ZMODE, int NWAVES, int MT, bool XLDS = false>
__global__ void __launch_bounds__(NWAVES * 64)
gemv_rows_mt(const uint16_t* __restrict__ x, const uint8_t* __restrict__ w,
             const uint16_t* __restrict__ scale, const uint16_t* __restrict__ zero,
             const uint16_t* __restrict__ bias, uint16_t* __restrict__ out, int M, int N, int K,
             int group_size, int gs_shift, int rows_per_block) {
  typedef typename TT<T>::storage S;
  static_assert(sizeof(S) == 2, "16-bit element types");
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  constexpr int NT = NWAVES * 64;
  constexpr int CK = BITS == 4 ? 128 : 64;
  constexpr int LK = CK / 4;
  constexpr int XV = LK / 8;
  const int nchunks = K / CK;
  const int row_bytes = nchunks * 64;
  const int G = K / group_size;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15;
  const int kb = lane >> 4;
  const int row0 = blockIdx.x * rows_per_block;
  int rows_blk = N - row0;
  if (rows_blk > rows_per_block) rows_blk = rows_per_block;
  if (rows_blk <= 0) return;
  const int ntiles = (rows_blk + 15) >> 4;

  // LDS: [red NWAVES*MT*256 f32 | the waves' x buffers (XLDS)][scales rows_per_block*G, padded
  //      to 16 B][zeros (asymmetric)]
  typedef RowsMtX<BITS, MT> XB;
  float* red = reinterpret_cast<float*>(smem);
  const int tile_bytes = (rows_per_block * G * 2 + 15) & ~15;
  constexpr size_t kRedBytes = (size_t)NWAVES * MT * 256 * 4;
  constexpr size_t kFront = XLDS && (size_t)NWAVES * XB::kWaveBytes > kRedBytes
                                ? (size_t)NWAVES * XB::kWaveBytes : kRedBytes;
  uint16_t* sl = reinterpret_cast<uint16_t*>(smem + kFront);
  uint16_t* zl = reinterpret_cast<uint16_t*>(reinterpret_cast<uint8_t*>(sl) + tile_bytes);
  uint8_t* xbuf = smem + (size_t)wave * XB::kWaveBytes;

  const uint8_t* wbase = w + (int64_t)row0 * row_bytes + kb * 16;
  auto issue = [&](int tile, int c, bool live) {
    const int row_l = tile * 16 + r;
    const bool ok = row_l < rows_blk;
    const uint8_t* q = wbase + (int64_t)(ok ? row_l : 0) * row_bytes + (int64_t)c * 64;
    return __builtin_nontemporal_load(
        reinterpret_cast<const u32x4*>(live ? q : w + (int64_t)row0 * row_bytes));
  };
  int c = wave;
  u32x4 cur = issue(0, c < nchunks ? c : 0, c < nchunks);

  const int tile_halves = rows_blk * G;
  const uint16_t* stile = scale + (int64_t)row0 * G;
  const uint16_t* ztile = ZMODE == kZeroAsym ? zero + (int64_t)row0 * G : stile;
  for (int e = tid; e < tile_halves; e += NT) {
    sl[e] = stile[e];
    if (ZMODE == kZeroAsym) zl[e] = ztile[e];
  }
  __syncthreads();

  // this lane's rows of x: row mt*16 + r of every tile (rows >= M feed outputs never stored and
  // re-read row 0), k-slot kb
  const uint8_t* xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int row = mt * 16 + r;
    xrow[mt] = reinterpret_cast<const uint8_t*>(x) + ((size_t)(row < M ? row : 0) * K + kb * LK) * 2;
  }
  // XLDS: request i of a chunk covers rows kRowsPerReq * i + lane / kLanesPerRow, 16 bytes per lane
  const uint8_t* xreq[XLDS ? XB::kReqs : 1];
  u32x4 xg[XLDS ? XB::kReqs : 1];
  if (XLDS) {
#pragma unroll
    for (int i = 0; i < XB::kReqs; ++i) {
      const int row = i * XB::kRowsPerReq + lane / XB::kLanesPerRow;
      xreq[i] = reinterpret_cast<const uint8_t*>(x) + (size_t)(row < M ? row : 0) * K * 2
                + (lane % XB::kLanesPerRow) * 16;
    }
  }
  auto request_x = [&](int chunk) {  // (a chunk past the end re-reads chunk 0)
#pragma unroll
    for (int i = 0; i < XB::kReqs; ++i) {
      xg[i] = *reinterpret_cast<const u32x4*>(xreq[i] + (size_t)chunk * XB::kRowBytes);
    }
  };
  if (XLDS) request_x(c < nchunks ? c : 0);
  f32x4 acc[kRowsMaxTiles][MT];
#pragma unroll
  for (int t = 0; t < kRowsMaxTiles; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  while (c < nchunks) {
    u32x4 xa[MT][XV];
    if (XLDS) {
      // the wave's own buffer: its LDS operations retire in order, so these stores cannot pass
      // the operand reads of the chunk before
#pragma unroll
      for (int i = 0; i < XB::kReqs; ++i) {
        const int row = i * XB::kRowsPerReq + lane / XB::kLanesPerRow;
        *reinterpret_cast<u32x4*>(xbuf + row * XB::kPitch + (lane % XB::kLanesPerRow) * 16) = xg[i];
      }
      request_x(c + NWAVES < nchunks ? c + NWAVES : 0);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
        for (int j = 0; j < XV; ++j) {
          xa[mt][j] = *reinterpret_cast<const u32x4*>(xbuf + (mt * 16 + r) * XB::kPitch
                                                      + kb * (LK * 2) + j * 16);
        }
      }
    } else {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const u32x4* xp = reinterpret_cast<const u32x4*>(xrow[mt] + (size_t)c * (CK * 2));
#pragma unroll
        for (int j = 0; j < XV; ++j) xa[mt][j] = xp[j];
      }
    }
    const int k0 = c * CK + kb * LK;
    const int grp = gs_shift >= 0 ? (k0 >> gs_shift) : (k0 / group_size);
#pragma unroll
    for (int t = 0; t < kRowsMaxTiles; ++t) {
      if (t < ntiles) {
        // codes of the next item first: the next tile of this chunk, else tile 0 of the wave's
        // next chunk
        const bool last_t = t + 1 >= ntiles;
        const int nc = last_t ? c + NWAVES : c;
        const bool live = nc < nchunks;
        const u32x4 nxt = issue(last_t ? 0 : t + 1, live ? nc : 0, live);
        const int srow = (t * 16 + r) * G;
        const float s = TT<T>::load(reinterpret_cast<const S*>(sl) + srow + grp);
        float z = 0.f;
        if (ZMODE == kZeroAsym) z = TT<T>::load(reinterpret_cast<const S*>(zl) + srow + grp);
        if (ZMODE == kZeroSymU) z = TT<T>::round(-(float)((1 << (BITS - 1)) - 1) * s);
        if constexpr (BITS == 4) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const u32x4 b = dequant8_b4<T, SIGNED, ZMODE>(cur[j], s, z);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[t][mt] = MfmaK32<T>::mma(xa[mt][j], b, acc[t][mt]);
          }
        } else {
          u32x4 b0, b1;
          dequant16_b8<T, SIGNED, ZMODE>(cur, s, z, b0, b1);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            acc[t][mt] = MfmaK32<T>::mma(xa[mt][0], b0, acc[t][mt]);
            acc[t][mt] = MfmaK32<T>::mma(xa[mt][1], b1, acc[t][mt]);
          }
        }
        cur = nxt;
      }
    }
    c += NWAVES;
  }

  // fold, one weight tile at a time: red[wave][m (MT*16)][n (16)]
  if (XLDS) __syncthreads();  // the reduction area overlays the x buffers of other waves
#pragma unroll
  for (int t = 0; t < kRowsMaxTiles; ++t) {
    if (t < ntiles) {
      if (t > 0) __syncthreads();  // the previous tile's sums have been read
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int m = mt * 16 + 4 * kb + v;
          red[(wave * (MT * 16) + m) * 16 + r] = acc[t][mt][v];
        }
      __syncthreads();
      for (int o = tid; o < M * 16; o += NT) {
        float sum = 0.f;
#pragma unroll
        for (int wv = 0; wv < NWAVES; ++wv) sum += red[wv * (MT * 256) + o];
        const int m = o >> 4;
        const int row_l = t * 16 + (o & 15);
        if (row_l < rows_blk) {
          if (bias != nullptr) sum += TT<T>::load(reinterpret_cast<const S*>(bias) + row0 + row_l);
          TT<T>::store(reinterpret_cast<S*>(out) + (int64_t)m * N + row0 + row_l, sum);
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// fp32 activations (the reference registers float next to half,
// groupwise_quantization_kernels.cu:844-851): the same row split on v_mfma_f32_16x16x4_f32, one
// fp32 value of x and one of w~ per lane and MFMA.  w~ = (float(q) * s) + z, both operations
// rounded to fp32 as in the reference; products and sums are fp32 inside the matrix core.
// x (m <= 16 rows) comes from L2.  Structure of gemv_rows_mt with a single tile of x.
// ---------------------------------------------------------------------------------------------
template<int BITS, bool SIGNED, int ZMODE, int NWAVES>
__global__ void __launch_bounds__(NWAVES * 64)
gemv_rows_f32(const float* __restrict__ x, const uint8_t* __restrict__ w,
              const float* __restrict__ scale, const float* __restrict__ zero,
              const float* __restrict__ bias, float* __restrict__ out, int M, int N, int K,
              int group_size, int gs_shift, int rows_per_block) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  constexpr int NT = NWAVES * 64;
  constexpr int CK = BITS == 4 ? 128 : 64;
  constexpr int LK = CK / 4;   // elements per lane and chunk
  constexpr int XV = LK / 4;   // 16-byte pieces of x per lane and chunk
  const int nchunks = K / CK;
  const int row_bytes = nchunks * 64;
  const int G = K / group_size;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15;
  const int kb = lane >> 4;
  const int row0 = blockIdx.x * rows_per_block;
  int rows_blk = N - row0;
  if (rows_blk > rows_per_block) rows_blk = rows_per_block;
  if (rows_blk <= 0) return;
  const int ntiles = (rows_blk + 15) >> 4;

  // LDS: [red NWAVES*256 f32][scales rows_per_block*G f32][zeros (asymmetric)]
  float* red = reinterpret_cast<float*>(smem);
  float* sl = red + NWAVES * 256;
  float* zl = sl + rows_per_block * G;

  const uint8_t* wbase = w + (int64_t)row0 * row_bytes + kb * 16;
  auto issue = [&](int tile, int c, bool live) {
    const int row_l = tile * 16 + r;
    const bool ok = row_l < rows_blk;
    const uint8_t* q = wbase + (int64_t)(ok ? row_l : 0) * row_bytes + (int64_t)c * 64;
    return __builtin_nontemporal_load(
        reinterpret_cast<const u32x4*>(live ? q : w + (int64_t)row0 * row_bytes));
  };
  int c = wave;
  u32x4 cur = issue(0, c < nchunks ? c : 0, c < nchunks);

  const int tile_elems = rows_blk * G;
  const float* stile = scale + (int64_t)row0 * G;
  const float* ztile = ZMODE == kZeroAsym ? zero + (int64_t)row0 * G : stile;
  for (int e = tid; e < tile_elems; e += NT) {
    sl[e] = stile[e];
    if (ZMODE == kZeroAsym) zl[e] = ztile[e];
  }
  __syncthreads();

  const float* xrow = x + (size_t)(r < M ? r : 0) * K + kb * LK;
  f32x4 acc[kRowsMaxTiles];
#pragma unroll
  for (int t = 0; t < kRowsMaxTiles; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

  while (c < nchunks) {
    f32x4 xa[XV];
#pragma unroll
    for (int j = 0; j < XV; ++j) xa[j] = reinterpret_cast<const f32x4*>(xrow + (size_t)c * CK)[j];
    const int k0 = c * CK + kb * LK;
    const int grp = gs_shift >= 0 ? (k0 >> gs_shift) : (k0 / group_size);
#pragma unroll
    for (int t = 0; t < kRowsMaxTiles; ++t) {
      if (t < ntiles) {
        const bool last_t = t + 1 >= ntiles;
        const int nc = last_t ? c + NWAVES : c;
        const bool live = nc < nchunks;
        const u32x4 nxt = issue(last_t ? 0 : t + 1, live ? nc : 0, live);
        const int srow = (t * 16 + r) * G;
        const float s = sl[srow + grp];
        float z = 0.f;
        if (ZMODE == kZeroAsym) z = zl[srow + grp];
        if (ZMODE == kZeroSymU) z = -(float)((1 << (BITS - 1)) - 1) * s;
        // a signed container is read as offset binary; the offset leaves inside the fused
        // multiply-add (u * s - off * s is exact before its single rounding)
        const float off = SIGNED ? -(float)(1 << (BITS - 1)) * s : 0.f;
#pragma unroll
        for (int wd = 0; wd < 4; ++wd) {
          uint32_t word = cur[wd];
          if (SIGNED) word ^= (BITS == 4 ? 0x88888888u : 0x80808080u);
          if constexpr (BITS == 4) {
            const uint32_t hi = (word >> 4) & 0x0F0F0F0Fu;  // elements 0, 2, 4, 6 of the word
            const uint32_t lo = word & 0x0F0F0F0Fu;         // elements 1, 3, 5, 7
#pragma unroll
            for (int b = 0; b < 4; ++b) {
              const float u0 = (float)((hi >> (8 * b)) & 0xFFu);
              const float u1 = (float)((lo >> (8 * b)) & 0xFFu);
              float w0 = SIGNED ? __builtin_fmaf(u0, s, off) : u0 * s;
              float w1 = SIGNED ? __builtin_fmaf(u1, s, off) : u1 * s;
              if (ZMODE != kZeroNone) {
                w0 = w0 + z;
                w1 = w1 + z;
              }
              // element 8*wd + 2*b (+1) of the lane's 32: piece 2*wd + b/2 of x, component 2*(b%2)
              acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(xa[2 * wd + (b >> 1)][2 * (b & 1)], w0,
                                                            acc[t], 0, 0, 0);
              acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(xa[2 * wd + (b >> 1)][2 * (b & 1) + 1],
                                                            w1, acc[t], 0, 0, 0);
            }
          } else {
#pragma unroll
            for (int b = 0; b < 4; ++b) {
              const float u0 = (float)((word >> (8 * b)) & 0xFFu);
              float w0 = SIGNED ? __builtin_fmaf(u0, s, off) : u0 * s;
              if (ZMODE != kZeroNone) w0 = w0 + z;
              acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(xa[wd][b], w0, acc[t], 0, 0, 0);
            }
          }
        }
        cur = nxt;
      }
    }
    c += NWAVES;
  }

  // fold, one weight tile at a time: red[wave][m (16)][n (16)]
#pragma unroll
  for (int t = 0; t < kRowsMaxTiles; ++t) {
    if (t < ntiles) {
      if (t > 0) __syncthreads();
#pragma unroll
      for (int v = 0; v < 4; ++v) red[(wave * 16 + 4 * kb + v) * 16 + r] = acc[t][v];
      __syncthreads();
      for (int o = tid; o < M * 16; o += NT) {
        float sum = 0.f;
#pragma unroll
        for (int wv = 0; wv < NWAVES; ++wv) sum += red[wv * 256 + o];
        const int m = o >> 4;
        const int row_l = t * 16 + (o & 15);
        if (row_l < rows_blk) {
          if (bias != nullptr) sum += bias[row0 + row_l];
          out[(int64_t)m * N + row0 + row_l] = sum;
        }
      }
    }
  }
}

inline size_t gemv_rows_f32_lds_bytes(int nwaves, int K, int group_size, int rows_per_block,
                                      bool asym) {
  const int G = K / group_size;
  return (size_t)nwaves * 256 * 4 + (size_t)(asym ? 2 : 1) * rows_per_block * G * 4;
}

inline size_t gemv_rows_mt_lds_bytes(int nwaves, int mt, int K, int group_size,
                                     int rows_per_block, bool asym, int bits = 4,
                                     bool xlds = false) {
  const int G = K / group_size;
  size_t front = (size_t)nwaves * mt * 256 * 4;
  const size_t xb = (size_t)nwaves * mt * 16 * ((bits == 4 ? 256 : 128) + 16);
  if (xlds && xb > front) front = xb;
  return front + (size_t)(asym ? 2 : 1) * ((rows_per_block * G * 2 + 15) & ~15);
}

inline size_t gemv_rows_lds_bytes(int nwaves, int M, int K, int group_size, int rows_per_block,
                                  bool asym, bool staged) {
  const int G = K / group_size;
  const size_t red = (size_t)((rows_per_block + 15) / 16) * nwaves * M * 16 * 4;
  const size_t xrows = staged ? (size_t)M * (K * 2 + 16) : 0;
  return (size_t)(asym ? 2 : 1) * ((rows_per_block * G * 2 + 15) & ~15) + 64
         + (red > xrows ? red : xrows);
}

}  // namespace
}  // namespace ofq
