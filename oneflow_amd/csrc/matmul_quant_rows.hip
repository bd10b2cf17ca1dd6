// matmul_quant with few rows of a (m <= 64 per pass): int8 x int8 on v_mfma_i32_16x16x64_i8 with
// the weights streamed from HBM once.
//
// The tiled GEMM needs 128-row tiles to earn its LDS traffic and leaves most CUs without a block
// when a has a handful of rows; here a block owns consecutive rows of b (about n / 256, at most
// 64, walked as 16-row tiles), a wave takes the 64-byte chunks c = wave, wave + NWAVES, ... of K,
// loads its 16 bytes of every 16-row tile of a straight from L2 and meets each weight tile with
// one MFMA per tile of a; the codes of the next (tile, chunk) are requested before the current
// ones are used.  int32 sums stay in registers, are added across the waves through LDS (integer
// addition: the order cannot matter) and leave through the epilogue of the GEMM path,
//   out = T(float(acc) * (a_scale * b_scale[n]) + bias[n]),
// so both paths give the same bits.
#include <atomic>
#include "ofq_device.h"
#include "ofq_internal.h"

namespace ofq {
namespace {

constexpr int kI8MaxTiles = 4;  // 16-row tiles of b per block

template<typename T, int NWAVES, int MT>
__global__ void __launch_bounds__(NWAVES * 64)
matmul_quant_rows(const uint8_t* __restrict__ a, const uint8_t* __restrict__ b,
                  const float* __restrict__ a_scale, const float* __restrict__ b_scale,
                  const typename TT<T>::storage* __restrict__ bias,
                  typename TT<T>::storage* __restrict__ out, int M, int N, int K,
                  int rows_per_block) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  constexpr int NT = NWAVES * 64;
  const int nchunks = K >> 6;
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
  int* red = reinterpret_cast<int*>(smem);  // [NWAVES][MT*16 (m)][16 (n)]

  const uint8_t* bbase = b + (int64_t)row0 * K + kb * 16;
  auto issue = [&](int tile, int c, bool live) {
    const int row_l = tile * 16 + r;
    const bool ok = row_l < rows_blk;
    const uint8_t* q = bbase + (int64_t)(ok ? row_l : 0) * K + (int64_t)c * 64;
    return __builtin_nontemporal_load(
        reinterpret_cast<const i32x4*>(live ? q : b + (int64_t)row0 * K));
  };
  int c = wave;
  i32x4 cur = issue(0, c < nchunks ? c : 0, c < nchunks);

  // this lane's rows of a: row mt*16 + r of every tile (rows >= M feed outputs never stored and
  // re-read row 0), bytes [16 kb, 16 kb + 16) of each chunk
  const uint8_t* arow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int row = mt * 16 + r;
    arow[mt] = a + (size_t)(row < M ? row : 0) * K + kb * 16;
  }
  i32x4 acc[kI8MaxTiles][MT];
#pragma unroll
  for (int t = 0; t < kI8MaxTiles; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = i32x4{0, 0, 0, 0};

  while (c < nchunks) {
    i32x4 av[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      av[mt] = *reinterpret_cast<const i32x4*>(arow[mt] + (size_t)c * 64);
#pragma unroll
    for (int t = 0; t < kI8MaxTiles; ++t) {
      if (t < ntiles) {
        const bool last_t = t + 1 >= ntiles;
        const int nc = last_t ? c + NWAVES : c;
        const bool live = nc < nchunks;
        const i32x4 nxt = issue(last_t ? 0 : t + 1, live ? nc : 0, live);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[t][mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(av[mt], cur, acc[t][mt], 0, 0, 0);
        cur = nxt;
      }
    }
    c += NWAVES;
  }

  const float sa = a_scale[0];
#pragma unroll
  for (int t = 0; t < kI8MaxTiles; ++t) {
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
        int sum = 0;
#pragma unroll
        for (int wv = 0; wv < NWAVES; ++wv) sum += red[wv * (MT * 256) + o];
        const int m = o >> 4;
        const int row_l = t * 16 + (o & 15);
        if (row_l < rows_blk) {
          const int n = row0 + row_l;
          float v = (float)sum * (sa * b_scale[n]);
          if (bias != nullptr) v = v + TT<T>::load(bias + n);
          TT<T>::store(out + (int64_t)m * N + n, v);
        }
      }
    }
  }
}

// ---- 1 to 4 rows of a: a wave owns whole rows of b -------------------------------------------
// With so few rows the matrix core adds nothing and its operand layout costs (a request of 16
// rows x 64 bytes instead of whole rows, a fold across the waves that split K).  Here lane l
// holds bytes [h * 1024 + 16 l, +16) of every row of a in registers (h < H = ceil(k / 1024)),
// a wave walks the rows w, w + NW, .. of the block's share of b with the requests of two rows in
// flight, meets each row with v_dot4_i32_i8 (exact int32) and sums across the lanes; no LDS, no
// barrier.  Same int32 sums and the same epilogue as the other paths, hence the same bits.
__device__ __forceinline__ int wave_sum_i32(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, false);   // quad_perm [1,0,3,2]
  v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, false);   // quad_perm [2,3,0,1]
  v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, false);  // row_half_mirror
  v += __builtin_amdgcn_update_dpp(0, v, 0x140, 0xF, 0xF, false);  // row_mirror
  return (__builtin_amdgcn_readlane(v, 0) + __builtin_amdgcn_readlane(v, 16))
         + (__builtin_amdgcn_readlane(v, 32) + __builtin_amdgcn_readlane(v, 48));
}

template<typename T, int NW, int H, int MR>
__global__ void __launch_bounds__(NW * 64)
matmul_quant_wave_rows(const uint8_t* __restrict__ a, const uint8_t* __restrict__ b,
                       const float* __restrict__ a_scale, const float* __restrict__ b_scale,
                       const typename TT<T>::storage* __restrict__ bias,
                       typename TT<T>::storage* __restrict__ out, int M, int N, int K,
                       int rows_per_block) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int row0 = blockIdx.x * rows_per_block;
  int rows_blk = N - row0;
  if (rows_blk > rows_per_block) rows_blk = rows_per_block;
  const int nr = rows_blk > wave ? (rows_blk - wave + NW - 1) / NW : 0;  // rows of this wave
  bool valid[H];
  uint32_t voff[H];
#pragma unroll
  for (int h = 0; h < H; ++h) {
    valid[h] = h * 1024 + lane * 16 < K;
    voff[h] = valid[h] ? (uint32_t)(h * 1024 + lane * 16) : 0u;
  }
  const uint8_t* bblk = b + (int64_t)row0 * K;
  i32x4 wq[2][H];
  auto issue = [&](int i, int buf) {
    const bool live = i < nr;  // the same for every lane
    const uint8_t* rowp = bblk + (size_t)(live ? wave + i * NW : 0) * K;
#pragma unroll
    for (int h = 0; h < H; ++h) {
      wq[buf][h] = __builtin_nontemporal_load(
          reinterpret_cast<const i32x4*>(rowp + (live ? voff[h] : 0u)));
    }
  };
  // the rows of a first (they come from L2 and every row of b needs them), then two rows of b
  i32x4 av[MR][H];
#pragma unroll
  for (int m = 0; m < MR; ++m) {
    const uint8_t* arow = a + (size_t)(m < M ? m : 0) * K;
#pragma unroll
    for (int h = 0; h < H; ++h) av[m][h] = *reinterpret_cast<const i32x4*>(arow + voff[h]);
  }
  issue(0, 0);
  issue(1, 1);
  const float sa = a_scale[0];
  auto finish = [&](int i, int buf) {
    const int n = row0 + wave + i * NW;
    const float sb = b_scale[n];
    float bv = 0.f;
    if (bias != nullptr) bv = TT<T>::load(bias + n);
#pragma unroll
    for (int m = 0; m < MR; ++m) {
      int acc = 0;
#pragma unroll
      for (int h = 0; h < H; ++h) {
        int part = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          part = __builtin_amdgcn_sdot4(av[m][h][j], wq[buf][h][j], part, false);
        }
        acc += valid[h] ? part : 0;
      }
      const int sum = wave_sum_i32(acc);
      if (lane == 0 && m < M) {
        float v = (float)sum * (sa * sb);
        if (bias != nullptr) v = v + bv;
        TT<T>::store(out + (int64_t)m * N + n, v);
      }
    }
  };
  for (int i = 0; i < nr; i += 2) {
    finish(i, 0);
    issue(i + 2, 0);
    if (i + 1 < nr) finish(i + 1, 1);
    issue(i + 3, 1);
  }
}

template<typename T, int H, int MR>
int launch_wave_rows_inst(hipStream_t st, const uint8_t* a, const uint8_t* b, const float* a_scale,
                          const float* b_scale, const void* bias, void* out, int m, int64_t n,
                          int64_t k) {
  typedef typename TT<T>::storage S;
  // A lane holds 4 H MR registers of a and 8 H of b: 16 waves (128 registers each) while that
  // fits, 8 waves (256 each) beyond, where the compiler would otherwise spill to scratch memory
  // (8192 x 8192, 2 rows).
  constexpr int NW = H * (4 * MR + 8) <= 100 ? 16 : 8;
  // 16 waves per CU, twice as many blocks from 128 rows per block on; a wave then walks its rows
  // two ahead
  int64_t grid = 256 * (16 / NW);
  if ((n + grid - 1) / grid >= 128) grid *= 2;
  int rpb = (int)((n + grid - 1) / grid);
  if (rpb < NW) rpb = NW;
  grid = (n + rpb - 1) / rpb;
  matmul_quant_wave_rows<T, NW, H, MR><<<(unsigned)grid, NW * 64, 0, st>>>(
      a, b, a_scale, b_scale, static_cast<const S*>(bias), static_cast<S*>(out), m, (int)n, (int)k,
      rpb);
  return ofq_check_launch();
}

// m <= 2 with 16 | k <= 8192, m <= 4 with k <= 4096 (the rows of a are held in registers: 4 H m
// of them).  Three and four rows of more than 4 KB run faster on the matrix-core kernel below
// (4096 x 8192, 4 rows: 14.5 us here, 9.4 us there).
template<typename T>
int launch_wave_rows(hipStream_t st, const uint8_t* a, const uint8_t* b, const float* a_scale,
                     const float* b_scale, const void* bias, void* out, int m, int64_t n,
                     int64_t k) {
  const int h = (int)((k + 1023) / 1024);
#define OFQ_WR(HV)                                                                             \
  case HV:                                                                                     \
    if (m == 1) return launch_wave_rows_inst<T, HV, 1>(st, a, b, a_scale, b_scale, bias, out, m, n, k); \
    if (m == 2) return launch_wave_rows_inst<T, HV, 2>(st, a, b, a_scale, b_scale, bias, out, m, n, k); \
    if constexpr (HV <= 4) {                                                                   \
      return launch_wave_rows_inst<T, HV, 4>(st, a, b, a_scale, b_scale, bias, out, m, n, k);  \
    } else {                                                                                   \
      return OFQ_ERR_UNSUPPORTED;                                                              \
    }
  switch (h) {
    OFQ_WR(1) OFQ_WR(2) OFQ_WR(3) OFQ_WR(4) OFQ_WR(5) OFQ_WR(6) OFQ_WR(7) OFQ_WR(8)
    default: return OFQ_ERR_UNSUPPORTED;
  }
#undef OFQ_WR
}

template<typename T, int NW, int MT>
int launch_inst(hipStream_t st, const uint8_t* a, const uint8_t* b, const float* a_scale,
                const float* b_scale, const void* bias, void* out, int m, int64_t n, int64_t k,
                int grid, int rpb) {
  typedef typename TT<T>::storage S;
  const size_t lds = (size_t)NW * MT * 256 * 4;
  auto kern = matmul_quant_rows<T, NW, MT>;
  if (lds > 64 * 1024) {
    static std::atomic<uint64_t> lds_allowed{0};  // devices on which the kernel's LDS limit is raised
    if (!ofq_allow_dynamic_lds(reinterpret_cast<const void*>(kern), (int)lds, lds_allowed)) return OFQ_ERR_LAUNCH;
  }
  kern<<<grid, NW * 64, lds, st>>>(a, b, a_scale, b_scale, static_cast<const S*>(bias),
                                   static_cast<S*>(out), m, (int)n, (int)k, rpb);
  return ofq_check_launch();
}

template<typename T>
int launch_part(hipStream_t st, const uint8_t* a, const uint8_t* b, const float* a_scale,
                const float* b_scale, const void* bias, void* out, int m, int64_t n, int64_t k) {
  if (m <= 4 && k <= 8192 && k % 16 == 0) {
    const int rc = launch_wave_rows<T>(st, a, b, a_scale, b_scale, bias, out, m, n, k);
    if (rc != OFQ_ERR_UNSUPPORTED) return rc;
  }
  constexpr int kCUs = 256;
  const int64_t max_rows = 16 * kI8MaxTiles;
  int64_t grid = kCUs;
  if ((n + grid - 1) / grid > max_rows) grid = (n + max_rows - 1) / max_rows;
  int rpb = (int)((n + grid - 1) / grid);
  if (rpb < 16) rpb = 16;
  grid = (n + rpb - 1) / rpb;
  if (m <= 16) return launch_inst<T, 16, 1>(st, a, b, a_scale, b_scale, bias, out, m, n, k, (int)grid, rpb);
  if (m <= 32) return launch_inst<T, 16, 2>(st, a, b, a_scale, b_scale, bias, out, m, n, k, (int)grid, rpb);
  return launch_inst<T, 16, 4>(st, a, b, a_scale, b_scale, bias, out, m, n, k, (int)grid, rpb);
}

}  // namespace

bool matmul_quant_rows_supported(int64_t m, int64_t n, int64_t k) {
  return m >= 1 && n >= 1 && k % 64 == 0 && k <= (1 << 24) && n <= 0x7FFFFFFF - 64;
}

// a [m,k], b [n,k] int8; any m, 64 rows of a per pass over b
int launch_matmul_quant_rows(hipStream_t st, const void* a, const void* b, const float* a_scale,
                             const float* b_scale, const void* bias, void* out, int out_dtype,
                             int64_t m, int64_t n, int64_t k) {
  const size_t esz = out_dtype == OFQ_F32 ? 4 : 2;
  for (int64_t m0 = 0; m0 < m; m0 += 64) {
    const int mp = (int)(m - m0 < 64 ? m - m0 : 64);
    const uint8_t* ap = static_cast<const uint8_t*>(a) + (size_t)m0 * k;
    void* op = static_cast<char*>(out) + (size_t)m0 * n * esz;
    const uint8_t* bp = static_cast<const uint8_t*>(b);
    int rc;
    switch (out_dtype) {
      case OFQ_F16: rc = launch_part<f16>(st, ap, bp, a_scale, b_scale, bias, op, mp, n, k); break;
      case OFQ_BF16: rc = launch_part<bf16>(st, ap, bp, a_scale, b_scale, bias, op, mp, n, k); break;
      case OFQ_F32: rc = launch_part<float>(st, ap, bp, a_scale, b_scale, bias, op, mp, n, k); break;
      default: return OFQ_ERR_BAD_DTYPE;
    }
    if (rc != OFQ_OK) return rc;
  }
  return OFQ_OK;
}

}  // namespace ofq
