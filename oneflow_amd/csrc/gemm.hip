// MFMA GEMMs for gfx950:
//   (1) fused_linear_with_groupwise_quantized_weight for m > 16: either the weight tile is
//       dequantised on its way into LDS and feeds fp16/bf16 MFMA (the fp16/bf16 copy of the
//       weight that the reference materialises for m > 8,
//       oneflow/core/functional/impl/quantization.cpp:341-350, then never touches HBM), cut
//       along K into separate blocks when a workspace for partial sums is given and the tiles
//       alone would not fill the chip; or, at large m with a workspace, the weight is
//       dequantised once and a copy-fed GEMM runs on it;
//   (2) matmul_quant: int8 x int8 -> int32 MFMA with a per-row/per-tensor scale epilogue.
//
// All are instances of one byte-oriented core (gemm_kernels.h).  A tile row is always 128 bytes
// of K (64 fp16/bf16 or 128 int8 elements), a k-step of the 32x32 MFMA consumes 32 of those bytes
// per row (16 bytes per lane), so the same LDS layout and fragment addressing serve every type.
// This file only picks tile shapes and fills parameter blocks.
#include "gemm_kernels.h"
#include "ofq_device.h"
#include "ofq_internal.h"

namespace ofq {

// Width of the weight tile under a 256-row tile of x.  The blocks run in rounds of one per CU;
// a round costs about in proportion to the tile width, so the candidate with the smallest
// (rounds x width) wins, the wider one on a tie (less L2 -> LDS traffic per MFMA).  384 (waves
// 4 x 2, 64 x 192 per wave: 12 MFMAs per 8 fragment reads) is open to the copy-fed GEMMs only and
// runs about a tenth faster per column than the narrower tiles on random operands (2048 x 11008
// x 4096 bf16: 163 us against 182 us for 352-wide tiles on 8 x 1 waves, whose waves read 12
// fragments per 11 MFMAs), which its cost is credited with; 192 turns the 258 or 344 tiles of
// m = 768 / 1024 at n = 11008 (two rounds of 128-wide tiles, the second nearly empty) into one
// round of 174 / 232: 160 -> 115 us in-tile.
int pick_tile_width(int64_t m, int64_t n, bool allow_wide) {
  const int64_t m_tiles = (m + 255) / 256;
  auto cost = [&](int64_t bn) { return ((m_tiles * ((n + bn - 1) / bn) + 255) / 256) * bn; };
  int best = 128;
  if (cost(192) <= cost(best)) best = 192;
  // 256 x 256 (copy-fed operands only): one round of 256 blocks where 128-wide tiles take two
  // (int8 4096 x 4096 x 4096: 101 -> 87 us; bf16 4096 x 4096 x 11008 behind the dequantised
  // weight: 410 -> 331 us, 8192 rows 1050 -> 750 us)
  if (allow_wide && cost(256) <= cost(best)) best = 256;
  if (allow_wide && cost(384) * 9 <= cost(best) * 10) best = 384;
  return best;
}

namespace {

// x[m,k] * wt[n,k]^T with both operands in T (the dequantised weight of the two-pass path)
template<typename T, class MF>
int launch_plain(hipStream_t st, const LinearArgs& a, const void* wt) {
  typedef typename TT<T>::storage S;
  typedef EpBias<T> EP;
  BCopyParams bp;
  bp.b = static_cast<const uint8_t*>(wt);
  bp.ldb = a.k * 2;
  bp.N = (int)a.n;
  typename EP::Params ep;
  ep.bias = static_cast<const S*>(a.bias);
  ep.out = static_cast<S*>(a.out);
  // 256-row tiles that would leave a quarter of the CUs without a block, where 128 x 128 tiles
  // give 192 to 512 blocks: those, on 8 waves (1024 x 4096 x 4096)
  const int64_t b256 = ((a.m + 255) / 256) * ((a.n + 127) / 128);
  const int64_t b128 = ((a.m + 127) / 128) * ((a.n + 127) / 128);
  if (b256 < 192 && b128 >= 192 && b128 <= 512) {
    return launch_core2<MF, B2Copy<128, 512>, EP, 128, 128, 4, 2>(st, a.x, a.k * 2, bp, ep, a.m,
                                                                  a.n, a.k / 64);
  }
  switch (pick_tile_width(a.m, a.n, true)) {
    case 384:
      return launch_core2<MF, B2Copy<384, 512>, EP, 256, 384, 4, 2>(st, a.x, a.k * 2, bp, ep, a.m,
                                                                    a.n, a.k / 64);
    case 256:
      return launch_core2<MF, B2Copy<256, 512>, EP, 256, 256, 4, 2>(st, a.x, a.k * 2, bp, ep, a.m,
                                                                    a.n, a.k / 64);
    case 192:
      return launch_core2<MF, B2Copy<192, 512>, EP, 256, 192, 4, 2>(st, a.x, a.k * 2, bp, ep, a.m,
                                                                    a.n, a.k / 64);
    default:
      return launch_core2<MF, B2Copy<128, 512>, EP, 256, 128, 4, 2>(st, a.x, a.k * 2, bp, ep, a.m,
                                                                    a.n, a.k / 64);
  }
}

// Few blocks (m small against the tile height, or few weight tiles): K is cut into `splits`
// slices that run as separate blocks, each writing fp32 partial sums of the whole output tile to
// its slice of the workspace; splitk_finalize adds the slices in order (so the result does not
// depend on scheduling), adds the bias and rounds to T once.
template<typename T, int VEC>
__global__ void __launch_bounds__(256)
splitk_finalize(const float* __restrict__ part, const typename TT<T>::storage* __restrict__ bias,
                typename TT<T>::storage* __restrict__ out, int64_t MN, int N, int splits) {
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * VEC;
  if (i >= MN) return;
  float acc[VEC];
  if constexpr (VEC == 4) {
    const f32x4 v = *reinterpret_cast<const f32x4*>(part + i);
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[e] = v[e];
    for (int sidx = 1; sidx < splits; ++sidx) {
      const f32x4 u = *reinterpret_cast<const f32x4*>(part + (int64_t)sidx * MN + i);
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[e] += u[e];
    }
  } else {
    acc[0] = part[i];
    for (int sidx = 1; sidx < splits; ++sidx) acc[0] += part[(int64_t)sidx * MN + i];
  }
  const int n = (int)(i % N);  // VEC divides N: the VEC elements share a row
  typename TT<T>::storage o[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    float v = acc[e];
    if (bias != nullptr) v += TT<T>::load(bias + n + e);
    TT<T>::store(&o[e], v);
  }
  if constexpr (VEC == 4) {
    *reinterpret_cast<u32x2*>(out + i) = *reinterpret_cast<const u32x2*>(o);
  } else {
    out[i] = o[0];
  }
}

// Slices of K for the in-tile path: as many as still fit the blocks into one resident round
// (256x128 tiles: one 8-wave block per CU; 128x128: two 4-wave blocks), each at least 4 k-tiles.
int wq_splits(const LinearArgs& a) {
  if (a.m >= 1024) return 1;  // two-pass territory
  const int64_t bm = a.m > 128 ? 256 : 128;
  const int64_t slots = a.m > 128 ? 256 : 512;
  const int64_t blocks = ((a.m + bm - 1) / bm) * ((a.n + 127) / 128);
  int64_t s = slots / blocks;
  const int64_t kt = a.k / 64;
  if (s > 8) s = 8;
  if (s > kt / 4) s = kt / 4;
  if (s < 1) s = 1;
  // no empty last slice
  while (s > 1 && ((kt + s - 1) / s) * (s - 1) >= kt) --s;
  return (int)s;
}

template<typename T, class MF, int BITS, bool SIGNED, int ZMODE>
int launch_wq_variant(hipStream_t st, const LinearArgs& a, float* partials, int splits) {
  typedef typename TT<T>::storage S;
  typedef EpBias<T> EP;
  WqParams<T> bp;
  bp.w = static_cast<const uint8_t*>(a.w);
  bp.scale = static_cast<const S*>(a.scale);
  bp.zero = static_cast<const S*>(a.zero);
  bp.ldw = a.k * BITS / 8;
  bp.N = (int)a.n;
  bp.G = (int)(a.k / a.group_size);
  bp.group_size = (int)a.group_size;
  typename EP::Params ep;
  ep.bias = static_cast<const S*>(a.bias);
  ep.out = static_cast<S*>(a.out);
  if (partials != nullptr && splits > 1) {
    EpPartial::Params pp;
    pp.out = partials;
    int rc;
    if (a.m > 128) {
      rc = launch_core2<MF, B2Dequant<T, BITS, SIGNED, ZMODE, 128, 512>, EpPartial, 256, 128, 4,
                        2>(st, a.x, a.k * 2, bp, pp, a.m, a.n, a.k / 64, splits);
    } else {
      // 8 waves on the 128x128 tile (32x64 per wave): more waves to hide the slice's short
      // k loop behind (28 us against 33 us on 4 waves at m = 128, 11008x4096)
      rc = launch_core2<MF, B2Dequant<T, BITS, SIGNED, ZMODE, 128, 512>, EpPartial, 128, 128, 4,
                        2>(st, a.x, a.k * 2, bp, pp, a.m, a.n, a.k / 64, splits);
    }
    if (rc != OFQ_OK) return rc;
    const int64_t mn = a.m * a.n;
    if (a.n % 4 == 0) {
      splitk_finalize<T, 4><<<(unsigned)((mn / 4 + 255) / 256), 256, 0, st>>>(
          partials, ep.bias, ep.out, mn, (int)a.n, splits);
    } else {
      splitk_finalize<T, 1><<<(unsigned)((mn + 255) / 256), 256, 0, st>>>(
          partials, ep.bias, ep.out, mn, (int)a.n, splits);
    }
    return ofq_check_launch();
  }
  // 256x128 tiles on 8 waves when there are enough rows of x to fill them, else 128x128 on 4
  if (a.m > 128) {
    if (pick_tile_width(a.m, a.n, false) == 192) {
      return launch_core2<MF, B2Dequant<T, BITS, SIGNED, ZMODE, 192, 512>, EP, 256, 192, 4, 2>(
          st, a.x, a.k * 2, bp, ep, a.m, a.n, a.k / 64);
    }
    return launch_core2<MF, B2Dequant<T, BITS, SIGNED, ZMODE, 128, 512>, EP, 256, 128, 4, 2>(
        st, a.x, a.k * 2, bp, ep, a.m, a.n, a.k / 64);
  }
  // few rows of x: 128-wide weight tiles would leave most CUs without a block (86 tiles for
  // n = 11008), so the weight tile shrinks until the grid covers the chip
  const int64_t n_tiles128 = (a.n + 127) / 128;
  if (n_tiles128 < 192) {
    return launch_core2<MF, B2Dequant<T, BITS, SIGNED, ZMODE, 32, 256>, EP, 128, 32, 4, 1>(
        st, a.x, a.k * 2, bp, ep, a.m, a.n, a.k / 64);
  }
  return launch_core2<MF, B2Dequant<T, BITS, SIGNED, ZMODE, 128, 256>, EP, 128, 128, 2, 2>(
      st, a.x, a.k * 2, bp, ep, a.m, a.n, a.k / 64);
}

template<typename T, class MF>
int launch_wq_t(hipStream_t st, const LinearArgs& a, float* partials, int splits) {
  const int zmode = !a.symmetric ? 2 : (a.w_signed ? 0 : 1);
#define OFQ_V(B, SG, ZM)                                       \
  if (a.bits == B && a.w_signed == SG && zmode == ZM)          \
    return launch_wq_variant<T, MF, B, SG, ZM>(st, a, partials, splits);
  OFQ_V(4, true, 0)
  OFQ_V(4, false, 1)
  OFQ_V(4, false, 2)
  OFQ_V(8, true, 0)
  OFQ_V(8, false, 1)
  OFQ_V(8, false, 2)
#undef OFQ_V
  return OFQ_ERR_UNSUPPORTED;
}

}  // namespace

bool gemm_wq_supported(const LinearArgs& a) {
  if (a.t_dtype != OFQ_F16 && a.t_dtype != OFQ_BF16) return false;
  if (a.group_dim != 1 || a.m < 1) return false;
  const int elems_per_chunk = a.bits == 4 ? 32 : 16;
  if (a.k % 64 != 0 || a.group_size % elems_per_chunk != 0) return false;
  return true;
}

// Two passes pay once m is large: the in-tile path converts every weight tile once per 256 rows
// of x (8 times at m = 2048) and that conversion, not the MFMAs, bounds it; converting the weight
// once into the workspace and running the copy-fed GEMM on it is what the reference functor does
// for m > 8 (oneflow/core/functional/impl/quantization.cpp:341-350).
size_t gemm_wq_workspace_bytes(const LinearArgs& a) {
  if (!gemm_wq_supported(a)) return 0;
  if (a.m >= 1024) return (size_t)a.n * (size_t)a.k * 2;
  const int splits = wq_splits(a);
  return splits > 1 ? (size_t)splits * (size_t)a.m * (size_t)a.n * 4 : 0;  // fp32 partial sums
}

int launch_gemm_wq(hipStream_t st, const LinearArgs& a, void* workspace, size_t workspace_bytes) {
  const size_t need = gemm_wq_workspace_bytes(a);
  const bool have_ws =
      need != 0 && workspace != nullptr && workspace_bytes >= need && ofq_aligned16(workspace);
  if (have_ws && a.m < 1024) {
    float* partials = static_cast<float*>(workspace);
    const int splits = wq_splits(a);
    if (a.t_dtype == OFQ_F16) return launch_wq_t<f16, MfmaF16>(st, a, partials, splits);
    return launch_wq_t<bf16, MfmaBF16>(st, a, partials, splits);
  }
  if (have_ws) {
    const int rc = ofq_groupwise_dequantize(st, a.w, a.scale, a.zero, workspace,
                                            a.w_signed ? OFQ_I8 : OFQ_U8, a.t_dtype, a.bits,
                                            a.symmetric ? 1 : 0, a.n * (a.k / a.group_size),
                                            a.group_size, 1);
    if (rc != OFQ_OK) return rc;
    if (a.t_dtype == OFQ_F16) return launch_plain<f16, MfmaF16>(st, a, workspace);
    return launch_plain<bf16, MfmaBF16>(st, a, workspace);
  }
  if (a.t_dtype == OFQ_F16) return launch_wq_t<f16, MfmaF16>(st, a, nullptr, 1);
  return launch_wq_t<bf16, MfmaBF16>(st, a, nullptr, 1);
}

// Groups along N: nothing to gain from converting inside the GEMM (a k-tile of a weight row would
// need 64 scales); above the streaming kernel's range the weight is dequantised once into the
// workspace -- the reference functor's own decomposition for m > 8,
// oneflow/core/functional/impl/quantization.cpp:341-350 -- and the copy-fed GEMM runs on it.
namespace {

// K slices of the copy-fed GEMM when its 256 x 128 tiles alone would leave most CUs without a
// block (m = 256 at n = 4096: 32 tiles): as many as fit one resident round, each >= 4 k-tiles
int gn_splits(const LinearArgs& a) {
  const int64_t blocks = ((a.m + 255) / 256) * ((a.n + 127) / 128);
  int64_t s = 256 / blocks;
  const int64_t kt = a.k / 64;
  if (s > 8) s = 8;
  if (s > kt / 4) s = kt / 4;
  if (s < 1) s = 1;
  while (s > 1 && ((kt + s - 1) / s) * (s - 1) >= kt) --s;  // no empty last slice
  return (int)s;
}

template<typename T, class MF>
int launch_plain_split(hipStream_t st, const LinearArgs& a, const void* wt, float* partials,
                       int splits) {
  typedef typename TT<T>::storage S;
  BCopyParams bp;
  bp.b = static_cast<const uint8_t*>(wt);
  bp.ldb = a.k * 2;
  bp.N = (int)a.n;
  EpPartial::Params pp;
  pp.out = partials;
  const int rc = launch_core2<MF, B2Copy<128, 512>, EpPartial, 256, 128, 4, 2>(
      st, a.x, a.k * 2, bp, pp, a.m, a.n, a.k / 64, splits);
  if (rc != OFQ_OK) return rc;
  const int64_t mn = a.m * a.n;
  const S* bias = static_cast<const S*>(a.bias);
  S* out = static_cast<S*>(a.out);
  if (a.n % 4 == 0) {
    splitk_finalize<T, 4><<<(unsigned)((mn / 4 + 255) / 256), 256, 0, st>>>(partials, bias, out, mn,
                                                                          (int)a.n, splits);
  } else {
    splitk_finalize<T, 1><<<(unsigned)((mn + 255) / 256), 256, 0, st>>>(partials, bias, out, mn,
                                                                      (int)a.n, splits);
  }
  return ofq_check_launch();
}

inline size_t round_up_256(size_t v) { return (v + 255) & ~(size_t)255; }

}  // namespace

// [dequantised weight n*k*sizeof(T), padded to 256 B][fp32 partial sums of the K slices, if any]
size_t gemm_gn_workspace_bytes(const LinearArgs& a) {
  if (a.group_dim != 0 || (a.t_dtype != OFQ_F16 && a.t_dtype != OFQ_BF16)) return 0;
  if (a.m <= 64 || a.k % 64 != 0 || a.n % a.group_size != 0) return 0;
  const int splits = gn_splits(a);
  return round_up_256((size_t)a.n * (size_t)a.k * 2)
         + (splits > 1 ? (size_t)splits * (size_t)a.m * (size_t)a.n * 4 : 0);
}

int launch_gemm_gn(hipStream_t st, const LinearArgs& a, void* workspace) {
  const int rc = ofq_groupwise_dequantize(st, a.w, a.scale, a.zero, workspace,
                                          a.w_signed ? OFQ_I8 : OFQ_U8, a.t_dtype, a.bits,
                                          a.symmetric ? 1 : 0, a.n / a.group_size, a.group_size,
                                          a.k);
  if (rc != OFQ_OK) return rc;
  const int splits = gn_splits(a);
  if (splits > 1) {
    float* partials = reinterpret_cast<float*>(static_cast<char*>(workspace)
                                               + round_up_256((size_t)a.n * (size_t)a.k * 2));
    if (a.t_dtype == OFQ_F16) {
      return launch_plain_split<f16, MfmaF16>(st, a, workspace, partials, splits);
    }
    return launch_plain_split<bf16, MfmaBF16>(st, a, workspace, partials, splits);
  }
  if (a.t_dtype == OFQ_F16) return launch_plain<f16, MfmaF16>(st, a, workspace);
  return launch_plain<bf16, MfmaBF16>(st, a, workspace);
}

}  // namespace ofq

using namespace ofq;

// rows of a up to which matmul_quant streams the weights instead of tiling them
static constexpr int64_t kMatmulQuantRowsMaxM = 64;

namespace ofq {
namespace {

// K slices of the int8 GEMM when its 128-wide tiles alone would leave most CUs without a block:
// as many as still fit one resident round (256x128 tiles: one block per CU; 128x128: two), each
// at least 4 k-tiles of 128.
// Tiles below 256 rows, one launch, no K slices and no workspace, for the int8 GEMM on rows of up
// to 6144 codes (a block's k loop costs about 0.4 us per 128-byte k-tile whatever the tile, so
// on long rows K slices win again: 256 x 4096 x 11008 46.9 us against 27.8 us):
//  - 64 x 64 tiles (4 waves) when there are 128 to 768 of them: they alone fill the chip
//    (256 x 4096 x 4096: 256 blocks) and no partial sum leaves it -- 13.3 us against 18.7 us with
//    slices; 128 rows 12.6 against 15.1, 512 rows 18.7 against 24.5, 768 rows 24.9 against 34.9,
//    256 x 11008 x 4096 23.1 against 33.1;
//  - 128 x 128 tiles on 8 waves when the 256-row tiles would leave a quarter of the CUs without
//    a block and these give 192 to 512 blocks (1024 x 4096 x 4096: 28.7 against 36.3 us,
//    512 x 11008 x 4096: 40.5 against 48.3 us).
enum MqTile { kMqTileDefault = 0, kMqTile64 = 64, kMqTile128 = 128 };
MqTile mq_tile(int64_t m, int64_t n, int64_t k) {
  if (m <= kMatmulQuantRowsMaxM || k % 128 != 0 || k > 6144) return kMqTileDefault;
  const int64_t t64 = ((m + 63) / 64) * ((n + 63) / 64);
  if (m <= 768 && t64 >= 128 && t64 <= 768) return kMqTile64;
  const int64_t b256 = ((m + 255) / 256) * ((n + 127) / 128);
  const int64_t b128 = ((m + 127) / 128) * ((n + 127) / 128);
  if (b256 < 192 && b128 >= 192 && b128 <= 512) return kMqTile128;
  return kMqTileDefault;
}

int mq_splits(int64_t m, int64_t n, int64_t k) {
  if (mq_tile(m, n, k) != kMqTileDefault) return 1;
  // long rows (k >= 8192) already pay for slices from 33 rows of a on: 4096 x 11008 at m = 64
  // streams in 33 us and runs in 22 us as slices
  if (m <= (k >= 8192 ? kMatmulQuantRowsMaxM / 2 : kMatmulQuantRowsMaxM) || k % 128 != 0) return 1;
  int64_t bm = m > 128 ? 256 : 128;
  int64_t slots = m > 128 ? 256 : 512;
  // up to 512 rows on a weight with few column tiles: 128-row tiles and fewer, longer slices
  // write half the partial sums (256 x 4096 x 4096: 21.2 -> 18.8 us, 128 rows: 18.2 -> 15.1 us)
  const bool few_tiles = m <= 512 && ((m + 127) / 128) * ((n + 127) / 128) <= 128;
  if (few_tiles) {
    bm = 128;
    slots = m <= 128 ? 128 : 256;
  }
  const int64_t blocks = ((m + bm - 1) / bm) * ((n + 127) / 128);
  int64_t s = slots / blocks;
  const int64_t kt = k / 128;
  if (s > 8) s = 8;
  if (s > kt / 4) s = kt / 4;
  if (s < 1) s = 1;
  while (s > 1 && ((kt + s - 1) / s) * (s - 1) >= kt) --s;  // no empty last slice
  return (int)s;
}

// adds the int32 slices (integer addition: any order gives the same sum) and applies the
// epilogue of EpScale
template<typename T, int VEC>
__global__ void __launch_bounds__(256)
splitk_finalize_i32(const int* __restrict__ part, const float* __restrict__ a_scale,
                    const float* __restrict__ b_scale,
                    const typename TT<T>::storage* __restrict__ bias,
                    typename TT<T>::storage* __restrict__ out, int64_t MN, int N, int splits) {
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * VEC;
  if (i >= MN) return;
  int acc[VEC];
  if constexpr (VEC == 4) {
    const i32x4 v = *reinterpret_cast<const i32x4*>(part + i);
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[e] = v[e];
    for (int sidx = 1; sidx < splits; ++sidx) {
      const i32x4 u = *reinterpret_cast<const i32x4*>(part + (int64_t)sidx * MN + i);
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[e] += u[e];
    }
  } else {
    acc[0] = part[i];
    for (int sidx = 1; sidx < splits; ++sidx) acc[0] += part[(int64_t)sidx * MN + i];
  }
  const int n = (int)(i % N);  // VEC divides N: the VEC elements share a row
  const float sa = a_scale[0];
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    float r = (float)acc[e] * (sa * b_scale[n + e]);
    if (bias != nullptr) r = r + TT<T>::load(bias + n + e);
    TT<T>::store(out + i + e, r);
  }
}

template<typename T>
int launch_mq_split(hipStream_t st, const void* a, const BCopyParams& bp, const float* a_scale,
                    const float* b_scale, const void* bias, void* out, int64_t m, int64_t n,
                    int64_t k, float* partials, int splits) {
  typedef typename TT<T>::storage S;
  EpPartialI32::Params pp;
  pp.out = partials;
  int rc;
  const bool few_tiles = m <= 512 && ((m + 127) / 128) * ((n + 127) / 128) <= 128;  // as mq_splits
  if (m > 128 && !few_tiles) {
    rc = launch_core2<MfmaI8, B2Copy<128, 512>, EpPartialI32, 256, 128, 4, 2>(st, a, k, bp, pp, m,
                                                                             n, k / 128, splits);
  } else {
    rc = launch_core2<MfmaI8, B2Copy<128, 512>, EpPartialI32, 128, 128, 4, 2>(st, a, k, bp, pp, m,
                                                                             n, k / 128, splits);
  }
  if (rc != OFQ_OK) return rc;
  const int64_t mn = m * n;
  const int* pi = reinterpret_cast<const int*>(partials);
  if (n % 4 == 0) {
    splitk_finalize_i32<T, 4><<<(unsigned)((mn / 4 + 255) / 256), 256, 0, st>>>(
        pi, a_scale, b_scale, static_cast<const S*>(bias), static_cast<S*>(out), mn, (int)n, splits);
  } else {
    splitk_finalize_i32<T, 1><<<(unsigned)((mn + 255) / 256), 256, 0, st>>>(
        pi, a_scale, b_scale, static_cast<const S*>(bias), static_cast<S*>(out), mn, (int)n, splits);
  }
  return ofq_check_launch();
}

}  // namespace
}  // namespace ofq

extern "C" size_t ofq_matmul_quant_workspace_bytes(int64_t m, int64_t n, int64_t k) {
  if (m <= 0 || n <= 0 || k <= 0) return 0;
  const int splits = ofq::mq_splits(m, n, k);
  return splits > 1 ? (size_t)splits * (size_t)m * (size_t)n * 4 : 0;
}

extern "C" int ofq_matmul_quant_ws(void* stream, const void* a, const void* b, const float* a_scale,
                                   const float* b_scale, const void* bias, void* out, int out_dtype,
                                   int64_t m, int64_t n, int64_t k, void* workspace,
                                   size_t workspace_bytes);

extern "C" int ofq_matmul_quant(void* stream, const void* a, const void* b, const float* a_scale,
                                const float* b_scale, const void* bias, void* out, int out_dtype,
                                int64_t m, int64_t n, int64_t k) {
  return ofq_matmul_quant_ws(stream, a, b, a_scale, b_scale, bias, out, out_dtype, m, n, k, nullptr,
                             0);
}

extern "C" int ofq_matmul_quant_ws(void* stream, const void* a, const void* b, const float* a_scale,
                                   const float* b_scale, const void* bias, void* out, int out_dtype,
                                   int64_t m, int64_t n, int64_t k, void* workspace,
                                   size_t workspace_bytes) {
  OFQ_RETURN_IF(out_dtype != OFQ_F16 && out_dtype != OFQ_BF16 && out_dtype != OFQ_F32,
                OFQ_ERR_BAD_DTYPE);
  OFQ_RETURN_IF(m < 0 || n < 0 || k <= 0, OFQ_ERR_BAD_SHAPE);
  if (m == 0 || n == 0) return OFQ_OK;
  const int64_t i32max = 0x7FFFFFFF;
  OFQ_RETURN_IF(m * k > i32max || n * k > i32max || m * n > i32max, OFQ_ERR_UNSUPPORTED);
  // rows are consumed in 64-byte chunks of K (streaming kernel) or 128-byte tiles (GEMM)
  OFQ_RETURN_IF(k % 64 != 0, OFQ_ERR_UNSUPPORTED);
  OFQ_RETURN_IF(a == nullptr || b == nullptr || a_scale == nullptr || b_scale == nullptr
                    || out == nullptr,
                OFQ_ERR_NULL_POINTER);
  OFQ_RETURN_IF(!ofq_aligned16(a) || !ofq_aligned16(b) || !ofq_aligned16(out), OFQ_ERR_MISALIGNED);
  hipStream_t st = static_cast<hipStream_t>(stream);
  BCopyParams bp;
  bp.b = static_cast<const uint8_t*>(b);
  bp.ldb = k;
  bp.N = (int)n;
  {
    const int splits = mq_splits(m, n, k);
    const size_t need = (size_t)splits * (size_t)m * (size_t)n * 4;
    if (splits > 1 && workspace != nullptr && workspace_bytes >= need && ofq_aligned16(workspace)) {
      float* part = static_cast<float*>(workspace);
      switch (out_dtype) {
        case OFQ_F16:
          return launch_mq_split<f16>(st, a, bp, a_scale, b_scale, bias, out, m, n, k, part, splits);
        case OFQ_BF16:
          return launch_mq_split<bf16>(st, a, bp, a_scale, b_scale, bias, out, m, n, k, part,
                                       splits);
        default:
          return launch_mq_split<float>(st, a, bp, a_scale, b_scale, bias, out, m, n, k, part,
                                        splits);
      }
    }
  }
  // few rows of a, or a K the GEMM's tiles do not divide: the weights stream once per 64 rows
  if ((m <= kMatmulQuantRowsMaxM || k % 128 != 0) && matmul_quant_rows_supported(m, n, k)) {
    return launch_matmul_quant_rows(st, a, b, a_scale, b_scale, bias, out, out_dtype, m, n, k);
  }
  OFQ_RETURN_IF(k % 128 != 0, OFQ_ERR_UNSUPPORTED);
#define OFQ_MQ(T)                                                                              \
  {                                                                                            \
    typedef EpScale<T> EP;                                                                     \
    EP::Params ep;                                                                             \
    ep.a_scale = a_scale;                                                                      \
    ep.b_scale = b_scale;                                                                      \
    ep.bias = static_cast<const TT<T>::storage*>(bias);                                        \
    ep.out = static_cast<TT<T>::storage*>(out);                                                \
    const MqTile tile = mq_tile(m, n, k);                                                      \
    if (tile == kMqTile64) {                                                                   \
      return launch_core2<MfmaI8, B2Copy<64, 256>, EP, 64, 64, 2, 2>(st, a, k, bp, ep, m, n,   \
                                                                    k / 128);                  \
    }                                                                                          \
    if (tile == kMqTile128) {                                                                  \
      return launch_core2<MfmaI8, B2Copy<128, 512>, EP, 128, 128, 4, 2>(st, a, k, bp, ep, m,   \
                                                                       n, k / 128);            \
    }                                                                                          \
    const int bn = m > 128 ? pick_tile_width(m, n, true) : 128;                                \
    if (bn == 256) {                                                                           \
      return launch_core2<MfmaI8, B2Copy<256, 512>, EP, 256, 256, 4, 2>(st, a, k, bp, ep, m,   \
                                                                        n, k / 128);           \
    }                                                                                          \
    if (bn == 384) {                                                                           \
      return launch_core2<MfmaI8, B2Copy<384, 512>, EP, 256, 384, 4, 2>(st, a, k, bp, ep, m,   \
                                                                        n, k / 128);           \
    }                                                                                          \
    if (bn == 192) {                                                                           \
      return launch_core2<MfmaI8, B2Copy<192, 512>, EP, 256, 192, 4, 2>(st, a, k, bp, ep, m,   \
                                                                        n, k / 128);           \
    }                                                                                          \
    if (m > 128) {                                                                             \
      return launch_core2<MfmaI8, B2Copy<128, 512>, EP, 256, 128, 4, 2>(st, a, k, bp, ep, m,   \
                                                                        n, k / 128);           \
    }                                                                                          \
    return launch_core2<MfmaI8, B2Copy<128, 256>, EP, 128, 128, 2, 2>(st, a, k, bp, ep, m, n,  \
                                                                      k / 128);                \
  }
  switch (out_dtype) {
    case OFQ_F16: OFQ_MQ(f16)
    case OFQ_BF16: OFQ_MQ(bf16)
    default: OFQ_MQ(float)
  }
#undef OFQ_MQ
}
