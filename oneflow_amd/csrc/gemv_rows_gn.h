// fused_linear_with_groupwise_quantized_weight with the groups along N (group_dim = 0: scale and
// zero of shape [N / group_size, K], one value per k shared by group_size consecutive weight
// rows; oneflow/user/kernels/groupwise_quantization_kernels.cu:795-803), m <= 64, fp16 / bf16.
//
// Row split and MFMA arrangement of gemv_rows_mt: a block owns consecutive weight rows and walks
// them as 16-row tiles, a wave takes chunks c = wave, wave + NWAVES, ... of K, the MT sixteen-row
// tiles of x come straight from L2, sums stay in registers.  What differs is where a scale comes
// from: 16 | group_size and blocks start at multiples of 16, so a 16-row tile lies inside ONE
// group, and the scale rows of the (few) groups a block touches are copied to LDS once; a lane
// then reads the scales of its own k-slot (the same for all 16 rows of the tile: an LDS
// broadcast) and applies them element by element (dequant8_b4_v / dequant16_b8_v), w~ formed
// with the reference's roundings.
#pragma once

#include "dequant_regs.h"
#include "gemv_rows.h"
#include "ofq_device.h"

namespace ofq {
namespace {

// XLDS: x through per-wave buffers in LDS, requested with neighbouring lanes on neighbouring
// bytes one chunk ahead (see gemv_rows_mt); the buffers share their memory with `red`.
template<typename T, int BITS, bool SIGNED, int ZMODE, int NWAVES, int MT, bool XLDS = false>
__global__ void __launch_bounds__(NWAVES * 64)
gemv_rows_gn(const uint16_t* __restrict__ x, const uint8_t* __restrict__ w,
             const uint16_t* __restrict__ scale, const uint16_t* __restrict__ zero,
             const uint16_t* __restrict__ bias, uint16_t* __restrict__ out, int M, int N, int K,
             int group_size, int rows_per_block) {
  typedef typename TT<T>::storage S;
  static_assert(sizeof(S) == 2, "16-bit element types");
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  constexpr int NT = NWAVES * 64;
  constexpr int CK = BITS == 4 ? 128 : 64;  // elements per chunk: 64 bytes of codes per row
  constexpr int LK = CK / 4;                // elements per lane and chunk
  constexpr int XV = LK / 8;                // 16-byte pieces of x (and of scales) per lane and chunk
  const int nchunks = K / CK;
  const int row_bytes = nchunks * 64;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15;
  const int kb = lane >> 4;
  const int row0 = blockIdx.x * rows_per_block;  // a multiple of 16
  int rows_blk = N - row0;
  if (rows_blk > rows_per_block) rows_blk = rows_per_block;
  if (rows_blk <= 0) return;
  const int ntiles = (rows_blk + 15) >> 4;
  const int g_first = row0 / group_size;
  const int ng = (row0 + rows_blk - 1) / group_size - g_first + 1;

  // LDS: [red NWAVES*MT*256 f32 | the waves' x buffers (XLDS)][scale rows of the block's groups,
  //      ng x K][zero rows (asymmetric)]
  typedef RowsMtX<BITS, MT> XB;
  float* red = reinterpret_cast<float*>(smem);
  constexpr size_t kRedBytes = (size_t)NWAVES * MT * 256 * 4;
  constexpr size_t kFront = XLDS && (size_t)NWAVES * XB::kWaveBytes > kRedBytes
                                ? (size_t)NWAVES * XB::kWaveBytes : kRedBytes;
  uint16_t* sl = reinterpret_cast<uint16_t*>(smem + kFront);
  uint16_t* zl = sl + (size_t)ng * K;
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

  {
    const int pieces = ng * (K >> 3);
    const u32x4* ssrc = reinterpret_cast<const u32x4*>(scale + (int64_t)g_first * K);
    const u32x4* zsrc = reinterpret_cast<const u32x4*>(
        (ZMODE == kZeroAsym ? zero : scale) + (int64_t)g_first * K);
    for (int e = tid; e < pieces; e += NT) {
      reinterpret_cast<u32x4*>(sl)[e] = ssrc[e];
      if (ZMODE == kZeroAsym) reinterpret_cast<u32x4*>(zl)[e] = zsrc[e];
    }
  }
  __syncthreads();

  // element offset of each tile's scale row in `sl` / `zl`, plus the lane's k-slot
  int srow[kRowsMaxTiles];
#pragma unroll
  for (int t = 0; t < kRowsMaxTiles; ++t) {
    const int first = row0 + t * 16 < N ? row0 + t * 16 : row0;
    srow[t] = (first / group_size - g_first) * K + kb * LK;
  }

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
#pragma unroll
    for (int t = 0; t < kRowsMaxTiles; ++t) {
      if (t < ntiles) {
        const bool last_t = t + 1 >= ntiles;
        const int nc = last_t ? c + NWAVES : c;
        const bool live = nc < nchunks;
        const u32x4 nxt = issue(last_t ? 0 : t + 1, live ? nc : 0, live);
        const u32x4* sp = reinterpret_cast<const u32x4*>(sl + srow[t] + c * CK);
        const u32x4* zp = reinterpret_cast<const u32x4*>(zl + srow[t] + c * CK);
        const u32x4 none = {0u, 0u, 0u, 0u};
        if constexpr (BITS == 4) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const u32x4 b = dequant8_b4_v<T, SIGNED, ZMODE>(cur[j], sp[j],
                                                            ZMODE == kZeroAsym ? zp[j] : none);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[t][mt] = MfmaK32<T>::mma(xa[mt][j], b, acc[t][mt]);
          }
        } else {
          u32x4 b0, b1;
          dequant16_b8_v<T, SIGNED, ZMODE>(cur, sp[0], sp[1], ZMODE == kZeroAsym ? zp[0] : none,
                                           ZMODE == kZeroAsym ? zp[1] : none, b0, b1);
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

// fp32 activations (the reference registers float next to half): the same on
// v_mfma_f32_16x16x4_f32, one fp32 value of x and one of w~ per lane and MFMA, 16 rows of x per
// pass; w~ = (float(q) * s_k) + z_k with both operations rounded to fp32 as in the reference.
template<int BITS, bool SIGNED, int ZMODE, int NWAVES>
__global__ void __launch_bounds__(NWAVES * 64)
gemv_rows_f32_gn(const float* __restrict__ x, const uint8_t* __restrict__ w,
                 const float* __restrict__ scale, const float* __restrict__ zero,
                 const float* __restrict__ bias, float* __restrict__ out, int M, int N, int K,
                 int group_size, int rows_per_block) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  constexpr int NT = NWAVES * 64;
  constexpr int CK = BITS == 4 ? 128 : 64;
  constexpr int LK = CK / 4;   // elements per lane and chunk
  constexpr int XV = LK / 4;   // 16-byte pieces of x (and of scales) per lane and chunk
  const int nchunks = K / CK;
  const int row_bytes = nchunks * 64;
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
  const int g_first = row0 / group_size;
  const int ng = (row0 + rows_blk - 1) / group_size - g_first + 1;

  // LDS: [red NWAVES*256 f32][scale rows ng x K f32][zero rows (asymmetric)]
  float* red = reinterpret_cast<float*>(smem);
  float* sl = red + NWAVES * 256;
  float* zl = sl + (size_t)ng * K;

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
  {
    const int pieces = ng * (K >> 2);
    const f32x4* ssrc = reinterpret_cast<const f32x4*>(scale + (int64_t)g_first * K);
    const f32x4* zsrc = reinterpret_cast<const f32x4*>(
        (ZMODE == kZeroAsym ? zero : scale) + (int64_t)g_first * K);
    for (int e = tid; e < pieces; e += NT) {
      reinterpret_cast<f32x4*>(sl)[e] = ssrc[e];
      if (ZMODE == kZeroAsym) reinterpret_cast<f32x4*>(zl)[e] = zsrc[e];
    }
  }
  __syncthreads();

  int srow[kRowsMaxTiles];
#pragma unroll
  for (int t = 0; t < kRowsMaxTiles; ++t) {
    const int first = row0 + t * 16 < N ? row0 + t * 16 : row0;
    srow[t] = (first / group_size - g_first) * K + kb * LK;
  }
  const float* xrow = x + (size_t)(r < M ? r : 0) * K + kb * LK;
  f32x4 acc[kRowsMaxTiles];
#pragma unroll
  for (int t = 0; t < kRowsMaxTiles; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

  while (c < nchunks) {
    f32x4 xa[XV];
#pragma unroll
    for (int j = 0; j < XV; ++j) xa[j] = reinterpret_cast<const f32x4*>(xrow + (size_t)c * CK)[j];
#pragma unroll
    for (int t = 0; t < kRowsMaxTiles; ++t) {
      if (t < ntiles) {
        const bool last_t = t + 1 >= ntiles;
        const int nc = last_t ? c + NWAVES : c;
        const bool live = nc < nchunks;
        const u32x4 nxt = issue(last_t ? 0 : t + 1, live ? nc : 0, live);
        const float* sp = sl + srow[t] + c * CK;
        const float* zp = zl + srow[t] + c * CK;
        constexpr float kOff = -(float)(1 << (BITS - 1));
        constexpr float kSymZ = -(float)((1 << (BITS - 1)) - 1);
        // element e of the lane's LK: piece e / 4, component e % 4 of x; product and sum are
        // rounded separately, as the reference's dequantisation does
        auto fma_elem = [&](int e, float u) {
#pragma clang fp contract(off)
          const float s = sp[e];
          float wv = SIGNED ? __builtin_fmaf(u, s, kOff * s) : u * s;
          if (ZMODE == kZeroAsym) wv = wv + zp[e];
          if (ZMODE == kZeroSymU) {
            const float zs = kSymZ * s;
            wv = wv + zs;
          }
          acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(xa[e >> 2][e & 3], wv, acc[t], 0, 0, 0);
        };
#pragma unroll
        for (int wd = 0; wd < 4; ++wd) {
          uint32_t word = cur[wd];
          if (SIGNED) word ^= (BITS == 4 ? 0x88888888u : 0x80808080u);
          if constexpr (BITS == 4) {
            const uint32_t hi = (word >> 4) & 0x0F0F0F0Fu;  // elements 0, 2, 4, 6 of the word
            const uint32_t lo = word & 0x0F0F0F0Fu;         // elements 1, 3, 5, 7
#pragma unroll
            for (int b = 0; b < 4; ++b) {
              fma_elem(8 * wd + 2 * b, (float)((hi >> (8 * b)) & 0xFFu));
              fma_elem(8 * wd + 2 * b + 1, (float)((lo >> (8 * b)) & 0xFFu));
            }
          } else {
#pragma unroll
            for (int b = 0; b < 4; ++b) fma_elem(4 * wd + b, (float)((word >> (8 * b)) & 0xFFu));
          }
        }
        cur = nxt;
      }
    }
    c += NWAVES;
  }

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

inline size_t gemv_rows_f32_gn_lds_bytes(int nwaves, int K, int group_size, int rows_per_block,
                                         bool asym);

// groups a block of `rows_per_block` rows (a multiple of 16, starting at a multiple of itself)
// can touch
inline int gemv_rows_gn_groups(int rows_per_block, int group_size) {
  if (group_size % rows_per_block == 0) return 1;
  if (rows_per_block % group_size == 0) return rows_per_block / group_size;
  return (rows_per_block + group_size - 2) / group_size + 1;
}

inline size_t gemv_rows_gn_lds_bytes(int nwaves, int mt, int K, int group_size, int rows_per_block,
                                     bool asym, int bits = 4, bool xlds = false) {
  size_t front = (size_t)nwaves * mt * 256 * 4;
  const size_t xb = (size_t)nwaves * mt * 16 * ((bits == 4 ? 256 : 128) + 16);
  if (xlds && xb > front) front = xb;
  return front + (size_t)(asym ? 2 : 1) * gemv_rows_gn_groups(rows_per_block, group_size) * K * 2;
}

inline size_t gemv_rows_f32_gn_lds_bytes(int nwaves, int K, int group_size, int rows_per_block,
                                         bool asym) {
  return (size_t)nwaves * 256 * 4
         + (size_t)(asym ? 2 : 1) * gemv_rows_gn_groups(rows_per_block, group_size) * K * 4;
}

}  // namespace
}  // namespace ofq
