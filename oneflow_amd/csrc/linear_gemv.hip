// fused_linear_with_groupwise_quantized_weight, decode side (m <= 16), for gfx950, plus the
// any-shape fallback and the op's C entry point.
//
// Semantics (oneflow/user/kernels/groupwise_quantization_kernels.cu:582-642, :760-839):
//   w~[n,k] = T(T(q[n,k]) * scale[n,g]) + zero[n,g]   (both operations round to T)
//   out[m,n] = T( sum_k x[m,k] * w~[n,k]  (fp32 accumulation)  + float(bias[n]) )
//
// Decode kernel.  The reference launches one 128-thread block per output element and so streams
// the weights m times.  Here the m <= 16 rows of x ride along as the second operand of a
// 16x16x32 MFMA whose first dimension is 16 weight rows, so the weights are read from HBM exactly
// once whatever m is, and the k-reduction happens inside the matrix core instead of in a
// cross-lane tree:
//   - a block owns 16 consecutive weight rows and all of K; its waves take K in interleaved
//     chunks of 128 (4-bit) / 64 (8-bit) elements, i.e. one 128-bit load per lane covering
//     16 rows x 64 bytes;
//   - lane (r = lane%16, kb = lane/16) loads 16 bytes of row r; its 32 (16) codes feed the
//     "k-slot kb" of 4 (2) MFMAs.  The MFMA sums over k-slots, so any assignment of k to
//     (slot, element) is valid as long as the x operand uses the same one;
//   - int4 -> fp16 without conversions: (word & 0x000F000F) | 0x64006400 is the half2
//     (1024+q_lo, 1024+q_hi); the nibbles 4 bits up give 1024+16q.  One packed add (or fma by
//     1/16) recovers the codes exactly; an int8 container is first xor-ed with 0x88888888 to
//     turn two's complement nibbles into offset binary.  The codes come out pairwise
//     (e1,e5),(e0,e4),(e3,e7),(e2,e6) and x is permuted to match with four v_perm_b32;
//   - w~ is then formed exactly as the reference does (packed fp16 multiply by the group scale,
//     packed add of the zero term), bit-compatible with groupwise_dequantize -- in every kernel
//     but the fp16 fast path for symmetric 4-bit codes in an int8 container (gemv_w4s_f16 and
//     gemv_w4p_f16 with EXACT = false), which scales the exact fp32 group sum instead and never
//     rounds q*scale to fp16 (~3e-4 rel-L2 from the composition);
//   - partial sums of the waves are combined through LDS, bias is added in fp32, one rounding
//     to T.
#include <atomic>
#include "gemv_kernels.h"
#include "gemv_rows.h"
#include "ofq_device.h"
#include "ofq_internal.h"

namespace ofq {
namespace {

// ---- any shape, any grouping: one wave per weight row and up to MT rows of x ----------------
// The fallback for what the streaming kernels do not take (k off their chunk grid, odd group
// sizes).  A wave owns weight row n, its lanes walk k (two adjacent codes of a byte per step for
// 4-bit weights, so that a wave's requests are 64 consecutive bytes of codes), every element is
// dequantised once with the reference's roundings and meets the rows m0 .. m0+MT-1 of x;
// indices are 32-bit (the entry point bounds m*k, n*k and m*n by 2^31).
template<typename T, int BITS, bool SIGNED, int MT>
__global__ void __launch_bounds__(256)
linear_generic(const typename TT<T>::storage* __restrict__ x, const uint8_t* __restrict__ w,
               const typename TT<T>::storage* __restrict__ scale,
               const typename TT<T>::storage* __restrict__ zero,
               const typename TT<T>::storage* __restrict__ bias,
               typename TT<T>::storage* __restrict__ out, int M, int N, int K, int group_dim,
               int group_size, int symmetric) {
  constexpr int E = BITS == 4 ? 2 : 1;
  const int lane = threadIdx.x & 63;
  const int n = (int)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int m0 = (int)blockIdx.y * MT;
  if (n >= N) return;
  float acc[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) acc[i] = 0.f;
  auto zero_term = [&](float s, int si) -> float {
    if (!symmetric) return TT<T>::load(zero + si);
    if (SIGNED) return 0.f;
    return TT<T>::round(-(float)((1 << (BITS - 1)) - 1) * s);
  };
  auto element = [&](int k, float s, float z) {
    const float q = (float)code_at<BITS, SIGNED>(w, (int64_t)n * K + k);
    const float wv = TT<T>::round(TT<T>::round(q * s) + z);
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      if (m0 + i < M) acc[i] = __builtin_fmaf(TT<T>::load(x + (m0 + i) * K + k), wv, acc[i]);
    }
  };
  if (group_dim == 1) {
    // group by group: scale and zero are the same for the whole wave (one broadcast request per
    // group instead of one per element, no division per element).  Items (group, step of 64*E
    // elements within it) are taken four at a time with all their requests issued before any is
    // used: a wave walks its row alone, and one memory round trip per item would bound it.
    const int G = K / group_size;
    const int spg = (group_size + 64 * E - 1) / (64 * E);  // steps per group
    const int items = G * spg;
    constexpr int B = 4;
    for (int it0 = 0; it0 < items; it0 += B) {
      float sv[B], zv[B];
      int kk[B][E];
      bool ok[B][E];
      int code[B][E];
      float xv[B][E][MT];
#pragma unroll
      for (int b = 0; b < B; ++b) {
        const int it = it0 + b < items ? it0 + b : items - 1;
        const int gi = it / spg;  // (the same for every lane)
        const int st = it - gi * spg;
        const int si = n * G + gi;
        sv[b] = TT<T>::load(scale + si);
        zv[b] = zero_term(sv[b], si);
        const int kend = (gi + 1) * group_size;
#pragma unroll
        for (int e = 0; e < E; ++e) {
          const int k = gi * group_size + st * 64 * E + lane * E + e;
          ok[b][e] = it0 + b < items && k < kend;
          kk[b][e] = ok[b][e] ? k : 0;
          code[b][e] = code_at<BITS, SIGNED>(w, (int64_t)n * K + kk[b][e]);
#pragma unroll
          for (int i = 0; i < MT; ++i) {
            xv[b][e][i] = TT<T>::load(x + (m0 + i < M ? m0 + i : m0) * K + kk[b][e]);
          }
        }
      }
#pragma unroll
      for (int b = 0; b < B; ++b) {
#pragma unroll
        for (int e = 0; e < E; ++e) {
          const float wv = TT<T>::round(TT<T>::round((float)code[b][e] * sv[b]) + zv[b]);
#pragma unroll
          for (int i = 0; i < MT; ++i) {
            if (ok[b][e] && m0 + i < M) acc[i] = __builtin_fmaf(xv[b][e][i], wv, acc[i]);
          }
        }
      }
    }
  } else {
    const int srow = (n / group_size) * K;
    for (int k0 = lane * E; k0 < K; k0 += 64 * E) {
#pragma unroll
      for (int e = 0; e < E; ++e) {
        const int k = k0 + e;
        if (k < K) {
          const float s = TT<T>::load(scale + srow + k);
          element(k, s, zero_term(s, srow + k));
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    const float sum = wave_reduce(acc[i], OpSum());
    if (lane == 0 && m0 + i < M) {
      float r = sum;
      if (bias != nullptr) r += TT<T>::load(bias + n);
      TT<T>::store(out + (m0 + i) * N + n, r);
    }
  }
}

template<typename T>
int launch_generic_t(hipStream_t st, const LinearArgs& a) {
  typedef typename TT<T>::storage S;
  if (a.group_size > 0x7FFFFFFF) return OFQ_ERR_UNSUPPORTED;
#define OFQ_G1(B, SG, MTV)                                                                   \
  {                                                                                          \
    dim3 grid((unsigned)((a.n + 3) / 4), (unsigned)((a.m + MTV - 1) / MTV));                 \
    linear_generic<T, B, SG, MTV><<<grid, 256, 0, st>>>(                                     \
        static_cast<const S*>(a.x), static_cast<const uint8_t*>(a.w),                        \
        static_cast<const S*>(a.scale), static_cast<const S*>(a.zero),                       \
        static_cast<const S*>(a.bias), static_cast<S*>(a.out), (int)a.m, (int)a.n, (int)a.k, \
        a.group_dim, (int)a.group_size, a.symmetric ? 1 : 0);                                \
    return ofq_check_launch();                                                               \
  }
#define OFQ_G(B, SG)                                                                         \
  if (a.bits == B && a.w_signed == SG) {                                                     \
    if (a.m == 1) OFQ_G1(B, SG, 1)                                                           \
    if (a.m <= 4) OFQ_G1(B, SG, 4)                                                           \
    OFQ_G1(B, SG, 8)                                                                         \
  }
  OFQ_G(4, false) OFQ_G(4, true) OFQ_G(8, false) OFQ_G(8, true)
#undef OFQ_G
#undef OFQ_G1
  return OFQ_ERR_UNSUPPORTED;
}

inline int ilog2_exact(int64_t v) {
  if (v <= 0 || (v & (v - 1)) != 0) return -1;
  int s = 0;
  while ((1LL << s) < v) ++s;
  return s;
}

// ---- fast path launcher (gemv_w4s_f16) ------------------------------------------------------
template<int NW, bool STAGED>
int launch_w4s_inst(hipStream_t st, const LinearArgs& a, size_t lds, int cpg_shift) {
  auto kern = gemv_w4s_f16<NW, 2, STAGED>;
  if (lds > 64 * 1024) return OFQ_ERR_UNSUPPORTED;
  const int grid = (int)((a.n + 15) / 16);
  kern<<<grid, NW * 64, lds, st>>>(static_cast<const f16*>(a.x), static_cast<const uint8_t*>(a.w),
                                  static_cast<const f16*>(a.scale),
                                  static_cast<const f16*>(a.bias), static_cast<f16*>(a.out),
                                  (int)a.m, (int)a.n, (int)a.k, (int)a.group_size, cpg_shift);
  return ofq_check_launch();
}

bool w4s_supported(const LinearArgs& a) {
  return a.t_dtype == OFQ_F16 && a.bits == 4 && a.w_signed && a.symmetric && a.group_dim == 1
         && a.m >= 1 && a.m <= 16 && a.k % 128 == 0 && a.group_size % 128 == 0
         && a.k <= (1 << 20) && a.n <= 0x7FFFFFFF - 16;
}

// Row-balanced kernel: grid = a whole number of blocks per CU (or one 16-row tile per block when
// n is small), rows_per_block <= 64.
template<int NW, bool EXACT, bool SIGNED, int ZMODE, bool TILED = false, int PH = 1>
int launch_w4p_inst(hipStream_t st, const LinearArgs& a, int grid, int rows_per_block, size_t lds,
                    int cpg_shift) {
  auto kern = gemv_w4p_f16<NW, 1, EXACT, SIGNED, ZMODE, TILED, PH>;
  static std::atomic<uint64_t> lds_allowed{0};  // devices on which the kernel's LDS limit is raised
  if (!ofq_allow_dynamic_lds(reinterpret_cast<const void*>(kern), 160 * 1024, lds_allowed)) return OFQ_ERR_LAUNCH;
  kern<<<grid, NW * 64, lds, st>>>(static_cast<const f16*>(a.x), static_cast<const uint8_t*>(a.w),
                                  static_cast<const f16*>(a.scale),
                                  static_cast<const f16*>(a.zero),
                                  static_cast<const f16*>(a.bias), static_cast<f16*>(a.out),
                                  (int)a.m, (int)a.n, (int)a.k, (int)a.group_size, cpg_shift,
                                  rows_per_block);
  return ofq_check_launch();
}

// 4-bit codes, fp16, groups along K in multiples of 128: what the row-balanced kernel takes
bool w4p_supported(const LinearArgs& a) {
  return a.t_dtype == OFQ_F16 && a.bits == 4 && a.group_dim == 1 && a.m >= 1 && a.m <= 16
         && a.k % 128 == 0 && a.group_size % 128 == 0 && a.k <= (1 << 20)
         && a.n <= 0x7FFFFFFF - 16 && (a.symmetric || !a.w_signed);
}

// The row split of the row-balanced kernel, a function of n alone (the tile-major weight copy is
// laid out by it): one block per CU of a 256-CU part when that keeps a block within 64 rows (a
// single 16-row tile per block when n is small), else two, else as many 64-row blocks as it takes.
void w4p_row_split(int64_t n, int64_t* grid_out, int* rows_per_block_out) {
  constexpr int kCUs = 256;
  const int64_t max_rows = 16 * kW4pMaxTiles;
  int64_t grid = kCUs;
  if ((n + grid - 1) / grid > max_rows) grid = 2 * kCUs;
  if ((n + grid - 1) / grid > max_rows) grid = (n + max_rows - 1) / max_rows;
  int rpb = (int)((n + grid - 1) / grid);
  if (rpb < 16) rpb = 16;
  *grid_out = (n + rpb - 1) / rpb;
  *rows_per_block_out = rpb;
}

// OFQ_ERR_UNSUPPORTED when the shape does not fit the row-balanced kernel
int launch_w4p(hipStream_t st, const LinearArgs& a, int cpg_shift, bool tiled) {
  constexpr int kCUs = 256;
  int64_t grid;
  int rpb;
  w4p_row_split(a.n, &grid, &rpb);
  const bool two_per_cu = grid > kCUs;
  const int nw = two_per_cu ? 8 : 16;
  // one thread folds one output of the block
  if ((int64_t)((rpb + 15) / 16) * a.m * 16 > nw * 64) return OFQ_ERR_UNSUPPORTED;
  const bool exact = !(a.symmetric && a.w_signed);
  const size_t lds_cap = (two_per_cu ? 80u : 160u) * 1024u;
  size_t lds = gemv_w4p_lds_bytes(nw, (int)a.m, (int)a.k, (int)a.group_size, rpb, exact,
                                  !a.symmetric);
  if (a.m * a.k / 16 > (int64_t)kGemvMaxUnits * nw * 64 || lds > lds_cap) {
    // m * k beyond one staging of x: two to four stagings, each of an equal part of the chunk
    // pairs of a row (one block per CU only)
    if (nw != 16) return OFQ_ERR_UNSUPPORTED;
    int phases = 0;
    for (int ph = 2; ph <= 4 && phases == 0; ++ph) {
      const int64_t part_units = a.m * gemv_w4p_phase_chunks((int)a.k, ph) * 8;
      lds = gemv_w4p_lds_bytes(nw, (int)a.m, (int)a.k, (int)a.group_size, rpb, exact,
                               !a.symmetric, 1, ph);
      if (part_units <= (int64_t)kGemvMaxUnits * nw * 64 && lds <= lds_cap) phases = ph;
    }
    if (phases == 0) return OFQ_ERR_UNSUPPORTED;
#define OFQ_W4PN(TL, PHV)                                                                    \
  if (tiled == TL && phases == PHV) {                                                        \
    if (!exact)                                                                              \
      return launch_w4p_inst<16, false, true, kZeroNone, TL, PHV>(st, a, (int)grid, rpb,     \
                                                                  lds, cpg_shift);           \
    if (a.symmetric)                                                                         \
      return launch_w4p_inst<16, true, false, kZeroSymU, TL, PHV>(st, a, (int)grid, rpb,     \
                                                                  lds, cpg_shift);           \
    return launch_w4p_inst<16, true, false, kZeroAsym, TL, PHV>(st, a, (int)grid, rpb, lds,  \
                                                                cpg_shift);                  \
  }
    OFQ_W4PN(false, 2) OFQ_W4PN(true, 2) OFQ_W4PN(false, 3) OFQ_W4PN(true, 3)
    OFQ_W4PN(false, 4) OFQ_W4PN(true, 4)
#undef OFQ_W4PN
  }
#define OFQ_W4P(NWV, TL)                                                                     \
  if (nw == NWV && tiled == TL) {                                                            \
    if (!exact)                                                                              \
      return launch_w4p_inst<NWV, false, true, kZeroNone, TL>(st, a, (int)grid, rpb, lds,    \
                                                              cpg_shift);                    \
    if (a.symmetric)                                                                         \
      return launch_w4p_inst<NWV, true, false, kZeroSymU, TL>(st, a, (int)grid, rpb, lds,    \
                                                              cpg_shift);                    \
    return launch_w4p_inst<NWV, true, false, kZeroAsym, TL>(st, a, (int)grid, rpb, lds,      \
                                                            cpg_shift);                      \
  }
  OFQ_W4P(16, false) OFQ_W4P(8, false) OFQ_W4P(16, true) OFQ_W4P(8, true)
#undef OFQ_W4P
  return OFQ_ERR_UNSUPPORTED;
}

// ---- natural-order row-balanced kernel (gemv_rows): fp16 / bf16, 4- and 8-bit ----------------
template<typename T, int BITS, bool SIGNED, int ZMODE, int NW, bool STAGED>
int launch_rows_inst(hipStream_t st, const LinearArgs& a, int grid, int rows_per_block,
                     size_t lds, int gs_shift) {
  auto kern = gemv_rows<T, BITS, SIGNED, ZMODE, NW, STAGED>;
  static std::atomic<uint64_t> lds_allowed{0};  // devices on which the kernel's LDS limit is raised
  if (!ofq_allow_dynamic_lds(reinterpret_cast<const void*>(kern), 160 * 1024, lds_allowed)) return OFQ_ERR_LAUNCH;
  kern<<<grid, NW * 64, lds, st>>>(
      static_cast<const uint16_t*>(a.x), static_cast<const uint8_t*>(a.w),
      static_cast<const uint16_t*>(a.scale), static_cast<const uint16_t*>(a.zero),
      static_cast<const uint16_t*>(a.bias), static_cast<uint16_t*>(a.out), (int)a.m, (int)a.n,
      (int)a.k, (int)a.group_size, gs_shift, rows_per_block);
  return ofq_check_launch();
}

bool rows_supported(const LinearArgs& a) {
  if (a.t_dtype != OFQ_F16 && a.t_dtype != OFQ_BF16) return false;
  if (a.bits != 4 && a.bits != 8) return false;
  const int ck = a.bits == 4 ? 128 : 64;
  return a.group_dim == 1 && a.m >= 1 && a.m <= 16 && a.k % ck == 0
         && a.group_size % (ck / 4) == 0 && a.k <= (1 << 20) && a.n <= 0x7FFFFFFF - 16
         && (a.symmetric || !a.w_signed);
}

template<typename T, int NW>
int launch_rows_t(hipStream_t st, const LinearArgs& a, int grid, int rpb, size_t lds,
                  bool staged) {
  const int gs_shift = ilog2_exact(a.group_size);
  const int zmode = !a.symmetric ? kZeroAsym : (a.w_signed ? kZeroNone : kZeroSymU);
#define OFQ_R(B, SG, ZM)                                              \
  if (a.bits == B && a.w_signed == SG && zmode == ZM)                 \
    return staged ? launch_rows_inst<T, B, SG, ZM, NW, true>(st, a, grid, rpb, lds, gs_shift) \
                  : launch_rows_inst<T, B, SG, ZM, NW, false>(st, a, grid, rpb, lds, gs_shift);
  OFQ_R(4, true, kZeroNone)
  OFQ_R(4, false, kZeroSymU)
  OFQ_R(4, false, kZeroAsym)
  OFQ_R(8, true, kZeroNone)
  OFQ_R(8, false, kZeroSymU)
  OFQ_R(8, false, kZeroAsym)
#undef OFQ_R
  return OFQ_ERR_UNSUPPORTED;
}

// OFQ_ERR_UNSUPPORTED when x does not fit the block's registers and LDS
int launch_rows(hipStream_t st, const LinearArgs& a) {
  constexpr int kCUs = 256;
  const int64_t max_rows = 16 * kRowsMaxTiles;
  int64_t grid = kCUs;
  if ((a.n + grid - 1) / grid > max_rows) grid = 2 * kCUs;
  if ((a.n + grid - 1) / grid > max_rows) grid = (a.n + max_rows - 1) / max_rows;
  int rpb = (int)((a.n + grid - 1) / grid);
  if (rpb < 16) rpb = 16;
  grid = (a.n + rpb - 1) / rpb;
  const bool two_per_cu = grid > kCUs;
  const int nw = two_per_cu ? 8 : 16;
  const size_t cap = (two_per_cu ? 80u : 160u) * 1024u;
  // x goes to LDS when it fits there and in the staging registers; else it is read from L2
  bool staged = a.m * a.k / 8 <= (int64_t)kRowsMaxUnits * nw * 64;
  // bf16 with 4-bit codes and a zero term is bound by the vector unit (eleven instructions per
  // element pair); staging more than 64 KB of x adds to that (11008 x 4096 at 16 rows: 16.0
  // against 15.2 us), where the 8-bit and the symmetric variants gain from it (fp16 W8: 14.2
  // against 15.3 us)
  if (a.t_dtype == OFQ_BF16 && a.bits == 4 && !(a.symmetric && a.w_signed)
      && a.m * a.k * 2 > 65536) {
    staged = false;
  }
  size_t lds = gemv_rows_lds_bytes(nw, (int)a.m, (int)a.k, (int)a.group_size, rpb,
                                   !a.symmetric, staged);
  if (staged && lds > cap) {
    staged = false;
    lds = gemv_rows_lds_bytes(nw, (int)a.m, (int)a.k, (int)a.group_size, rpb, !a.symmetric,
                              false);
  }
  if (lds > cap) return OFQ_ERR_UNSUPPORTED;
  if (a.t_dtype == OFQ_BF16) {
    return nw == 16 ? launch_rows_t<bf16, 16>(st, a, (int)grid, rpb, lds, staged)
                    : launch_rows_t<bf16, 8>(st, a, (int)grid, rpb, lds, staged);
  }
  return nw == 16 ? launch_rows_t<f16, 16>(st, a, (int)grid, rpb, lds, staged)
                  : launch_rows_t<f16, 8>(st, a, (int)grid, rpb, lds, staged);
}

int launch_w4s(hipStream_t st, const LinearArgs& a) {
  const int64_t tiles = (a.n + 15) / 16;
  const int npairs = (int)((a.k / 128 + 1) / 2);
  const int cpg_shift = ilog2_exact(a.group_size / 128);
  // waves per block: as many as still let every block be resident at once (<= 24 waves per CU on
  // 256 CUs), so the kernel runs as a single round of blocks; never more than there are pairs
  // and never fewer than fold the block's m * 16 outputs with one thread each
  const int nw_min = a.m > 8 ? 4 : 2;
  int nw = 16;
  while (nw > nw_min && (tiles * nw > 6144 || nw > npairs)) nw >>= 1;
  const int nt = nw * 64;
  const int64_t nunits = a.m * a.k / 16;
  bool staged = nunits <= (int64_t)kGemvMaxUnits * nt;
  size_t lds = gemv_w4s_lds_bytes(nw, staged, (int)a.m, (int)a.k, (int)a.group_size);
  if (staged && lds > 48 * 1024) {
    staged = false;
    lds = gemv_w4s_lds_bytes(nw, false, (int)a.m, (int)a.k, (int)a.group_size);
  }
  // More than one 16-row tile per CU, or an x too large to stage per 16 rows: the row-balanced
  // kernel (equal bytes per block, x staged once per block) is the faster one.
  if (tiles > 256 || !staged) {
    int rc = launch_w4p(st, a, cpg_shift, false);
    if (rc != OFQ_ERR_UNSUPPORTED) return rc;
    // x too large for either staged kernel: the natural-order kernel reads x from L2 once per
    // block, the one below once per 16 rows
    if (!staged) {
      rc = launch_rows(st, a);
      if (rc != OFQ_ERR_UNSUPPORTED) return rc;
    }
  }
#define OFQ_W4S(NWV)                                                                   \
  if (nw == NWV)                                                                       \
    return staged ? launch_w4s_inst<NWV, true>(st, a, lds, cpg_shift)                  \
                  : launch_w4s_inst<NWV, false>(st, a, lds, cpg_shift);
  OFQ_W4S(16) OFQ_W4S(8) OFQ_W4S(4) OFQ_W4S(2)
#undef OFQ_W4S
  return OFQ_ERR_UNSUPPORTED;
}

template<int BITS, bool SIGNED, int ZMODE>
int launch_gemv_variant(hipStream_t st, const LinearArgs& a) {
  constexpr int CH = BITS == 4 ? 128 : 64;
  const int nchunks = (int)(a.k / CH);
  const int grid = (int)((a.n + 15) / 16);
  const int gs_shift = ilog2_exact(a.group_size);
  const f16* x = static_cast<const f16*>(a.x);
  const uint8_t* w = static_cast<const uint8_t*>(a.w);
  const f16* sc = static_cast<const f16*>(a.scale);
  const f16* ze = static_cast<const f16*>(a.zero);
  const f16* bi = static_cast<const f16*>(a.bias);
  f16* out = static_cast<f16*>(a.out);
  // waves per block: enough to spread K, few enough that every wave has >= 2 chunks
  if (nchunks >= 64) {
    gemv_f16_mfma<BITS, SIGNED, ZMODE, 16, 2><<<grid, 16 * 64, 0, st>>>(
        x, w, sc, ze, bi, out, (int)a.m, (int)a.n, (int)a.k, (int)a.group_size, gs_shift);
  } else if (nchunks >= 16) {
    gemv_f16_mfma<BITS, SIGNED, ZMODE, 8, 4><<<grid, 8 * 64, 0, st>>>(
        x, w, sc, ze, bi, out, (int)a.m, (int)a.n, (int)a.k, (int)a.group_size, gs_shift);
  } else {
    gemv_f16_mfma<BITS, SIGNED, ZMODE, 4, 2><<<grid, 4 * 64, 0, st>>>(
        x, w, sc, ze, bi, out, (int)a.m, (int)a.n, (int)a.k, (int)a.group_size, gs_shift);
  }
  return ofq_check_launch();
}

// ---- 16 < m <= 128: several tiles of x per weight tile ----------------------------------------
template<typename T, int BITS, bool SIGNED, int ZMODE, int NW, int MT, bool XLDS>
int launch_rows_mt_inst(hipStream_t st, const LinearArgs& a, const void* x, void* out, int m,
                        int grid, int rows_per_block, size_t lds) {
  auto kern = gemv_rows_mt<T, BITS, SIGNED, ZMODE, NW, MT, XLDS>;
  static std::atomic<uint64_t> lds_allowed{0};  // devices on which the kernel's LDS limit is raised
  if (!ofq_allow_dynamic_lds(reinterpret_cast<const void*>(kern), 160 * 1024, lds_allowed)) return OFQ_ERR_LAUNCH;
  kern<<<grid, NW * 64, lds, st>>>(
      static_cast<const uint16_t*>(x), static_cast<const uint8_t*>(a.w),
      static_cast<const uint16_t*>(a.scale), static_cast<const uint16_t*>(a.zero),
      static_cast<const uint16_t*>(a.bias), static_cast<uint16_t*>(out), m, (int)a.n, (int)a.k,
      (int)a.group_size, ilog2_exact(a.group_size), rows_per_block);
  return ofq_check_launch();
}

template<typename T, int NW, int MT, bool XLDS>
int launch_rows_mt_t(hipStream_t st, const LinearArgs& a, const void* x, void* out, int m,
                     int grid, int rpb, size_t lds) {
  const int zmode = !a.symmetric ? kZeroAsym : (a.w_signed ? kZeroNone : kZeroSymU);
#define OFQ_R(B, SG, ZM)                                              \
  if (a.bits == B && a.w_signed == SG && zmode == ZM)                 \
    return launch_rows_mt_inst<T, B, SG, ZM, NW, MT, XLDS>(st, a, x, out, m, grid, rpb, lds);
  OFQ_R(4, true, kZeroNone)
  OFQ_R(4, false, kZeroSymU)
  OFQ_R(4, false, kZeroAsym)
  OFQ_R(8, true, kZeroNone)
  OFQ_R(8, false, kZeroSymU)
  OFQ_R(8, false, kZeroAsym)
#undef OFQ_R
  return OFQ_ERR_UNSUPPORTED;
}

// rows [m0, m0 + m) of x, m <= 64
int launch_rows_mt_part(hipStream_t st, const LinearArgs& a, int64_t m0, int m) {
  constexpr int kCUs = 256;
  const int64_t max_rows = 16 * kRowsMaxTiles;
  int64_t grid = kCUs;
  if ((a.n + grid - 1) / grid > max_rows) grid = (a.n + max_rows - 1) / max_rows;
  int rpb = (int)((a.n + grid - 1) / grid);
  if (rpb < 16) rpb = 16;
  grid = (a.n + rpb - 1) / rpb;
  const int mt = (m + 15) / 16;  // 2, 3 or 4 tiles of x
  const size_t esz = 2;
  const void* x = static_cast<const char*>(a.x) + (size_t)m0 * a.k * esz;
  void* out = static_cast<char*>(a.out) + (size_t)m0 * a.n * esz;
  // x through per-wave buffers in LDS (coalesced requests, one chunk ahead): 12 waves for two
  // tiles of x, 8 for three and four (the buffers and the registers of the chunk in flight)
  {
    const int nw = mt == 2 ? 12 : 8;
    const size_t lds = gemv_rows_mt_lds_bytes(nw, mt, (int)a.k, (int)a.group_size, rpb,
                                              !a.symmetric, a.bits, true);
    if (lds <= 160u * 1024u) {
#define OFQ_MTX(TT_)                                                                            \
  switch (mt) {                                                                                 \
    case 2: return launch_rows_mt_t<TT_, 12, 2, true>(st, a, x, out, m, (int)grid, rpb, lds);   \
    case 3: return launch_rows_mt_t<TT_, 8, 3, true>(st, a, x, out, m, (int)grid, rpb, lds);    \
    default: return launch_rows_mt_t<TT_, 8, 4, true>(st, a, x, out, m, (int)grid, rpb, lds);   \
  }
      if (a.t_dtype == OFQ_BF16) { OFQ_MTX(bf16) }
      OFQ_MTX(f16)
#undef OFQ_MTX
    }
  }
  // x straight from L2 (the scales of a long-rowed block leave no room for the buffers):
  // 16 waves while the registers allow four waves per SIMD, 12 beyond
  const int nw = mt == 2 ? 16 : 12;
  const size_t lds =
      gemv_rows_mt_lds_bytes(nw, mt, (int)a.k, (int)a.group_size, rpb, !a.symmetric);
  if (lds > 160u * 1024u) return OFQ_ERR_UNSUPPORTED;
#define OFQ_MT(TT_)                                                                               \
  switch (mt) {                                                                                   \
    case 2: return launch_rows_mt_t<TT_, 16, 2, false>(st, a, x, out, m, (int)grid, rpb, lds);    \
    case 3: return launch_rows_mt_t<TT_, 12, 3, false>(st, a, x, out, m, (int)grid, rpb, lds);    \
    default: return launch_rows_mt_t<TT_, 12, 4, false>(st, a, x, out, m, (int)grid, rpb, lds);   \
  }
  if (a.t_dtype == OFQ_BF16) { OFQ_MT(bf16) }
  OFQ_MT(f16)
#undef OFQ_MT
}

// ---- fp32 activations -------------------------------------------------------------------------
template<int BITS, bool SIGNED, int ZMODE>
int launch_rows_f32_inst(hipStream_t st, const LinearArgs& a, const float* x, float* out, int m,
                         int grid, int rows_per_block, size_t lds) {
  auto kern = gemv_rows_f32<BITS, SIGNED, ZMODE, 16>;
  static std::atomic<uint64_t> lds_allowed{0};  // devices on which the kernel's LDS limit is raised
  if (!ofq_allow_dynamic_lds(reinterpret_cast<const void*>(kern), 160 * 1024, lds_allowed)) return OFQ_ERR_LAUNCH;
  kern<<<grid, 16 * 64, lds, st>>>(x, static_cast<const uint8_t*>(a.w),
                                  static_cast<const float*>(a.scale),
                                  static_cast<const float*>(a.zero),
                                  static_cast<const float*>(a.bias), out, m, (int)a.n, (int)a.k,
                                  (int)a.group_size, ilog2_exact(a.group_size), rows_per_block);
  return ofq_check_launch();
}

bool rows_f32_supported(const LinearArgs& a) {
  if (a.t_dtype != OFQ_F32 || (a.bits != 4 && a.bits != 8)) return false;
  const int ck = a.bits == 4 ? 128 : 64;
  return a.group_dim == 1 && a.m >= 1 && a.k % ck == 0 && a.group_size % (ck / 4) == 0
         && a.k <= (1 << 20) && a.n <= 0x7FFFFFFF - 16 && (a.symmetric || !a.w_signed);
}

// any m: 16 rows of x per pass over the weights
int launch_rows_f32(hipStream_t st, const LinearArgs& a) {
  constexpr int kCUs = 256;
  const int64_t max_rows = 16 * kRowsMaxTiles;
  int64_t grid = kCUs;
  if ((a.n + grid - 1) / grid > max_rows) grid = (a.n + max_rows - 1) / max_rows;
  int rpb = (int)((a.n + grid - 1) / grid);
  if (rpb < 16) rpb = 16;
  grid = (a.n + rpb - 1) / rpb;
  const size_t lds =
      gemv_rows_f32_lds_bytes(16, (int)a.k, (int)a.group_size, rpb, !a.symmetric);
  if (lds > 160u * 1024u) return OFQ_ERR_UNSUPPORTED;
  const int zmode = !a.symmetric ? kZeroAsym : (a.w_signed ? kZeroNone : kZeroSymU);
  for (int64_t m0 = 0; m0 < a.m; m0 += 16) {
    const int m = (int)(a.m - m0 < 16 ? a.m - m0 : 16);
    const float* x = static_cast<const float*>(a.x) + m0 * a.k;
    float* out = static_cast<float*>(a.out) + m0 * a.n;
    int rc = OFQ_ERR_UNSUPPORTED;
#define OFQ_R(B, SG, ZM)                                              \
  if (a.bits == B && a.w_signed == SG && zmode == ZM)                 \
    rc = launch_rows_f32_inst<B, SG, ZM>(st, a, x, out, m, (int)grid, rpb, lds);
    OFQ_R(4, true, kZeroNone)
    OFQ_R(4, false, kZeroSymU)
    OFQ_R(4, false, kZeroAsym)
    OFQ_R(8, true, kZeroNone)
    OFQ_R(8, false, kZeroSymU)
    OFQ_R(8, false, kZeroAsym)
#undef OFQ_R
    if (rc != OFQ_OK) return rc;
  }
  return OFQ_OK;
}

// ---- several problems, one launch -------------------------------------------------------------
template<typename T, int BITS, bool SIGNED, int ZMODE, int NW, bool STAGED>
int launch_rows_grouped_inst(hipStream_t st, const GemvGroup& g, int grid, int m, int k,
                             int group_size, int rows_per_block, size_t lds) {
  auto kern = gemv_rows_grouped<T, BITS, SIGNED, ZMODE, NW, STAGED>;
  static std::atomic<uint64_t> lds_allowed{0};  // devices on which the kernel's LDS limit is raised
  if (!ofq_allow_dynamic_lds(reinterpret_cast<const void*>(kern), 160 * 1024, lds_allowed)) return OFQ_ERR_LAUNCH;
  kern<<<grid, NW * 64, lds, st>>>(g, m, k, group_size, ilog2_exact(group_size), rows_per_block);
  return ofq_check_launch();
}

template<typename T, int NW, bool STAGED>
int launch_rows_grouped_t(hipStream_t st, const LinearArgs& a, const GemvGroup& g, int grid,
                          int rpb, size_t lds) {
  const int zmode = !a.symmetric ? kZeroAsym : (a.w_signed ? kZeroNone : kZeroSymU);
#define OFQ_R(B, SG, ZM)                                                           \
  if (a.bits == B && a.w_signed == SG && zmode == ZM)                              \
    return launch_rows_grouped_inst<T, B, SG, ZM, NW, STAGED>(st, g, grid, (int)a.m, (int)a.k, \
                                                              (int)a.group_size, rpb, lds);
  OFQ_R(4, true, kZeroNone)
  OFQ_R(4, false, kZeroSymU)
  OFQ_R(4, false, kZeroAsym)
  OFQ_R(8, true, kZeroNone)
  OFQ_R(8, false, kZeroSymU)
  OFQ_R(8, false, kZeroAsym)
#undef OFQ_R
  return OFQ_ERR_UNSUPPORTED;
}

template<int NW, bool EXACT, bool SIGNED, int ZMODE, int PH = 1>
int launch_w4p_grouped_inst(hipStream_t st, const GemvGroup& g, int grid, int m, int k,
                            int group_size, int rows_per_block, size_t lds) {
  auto kern = gemv_w4p_f16_grouped<NW, EXACT, SIGNED, ZMODE, PH>;
  static std::atomic<uint64_t> lds_allowed{0};  // devices on which the kernel's LDS limit is raised
  if (!ofq_allow_dynamic_lds(reinterpret_cast<const void*>(kern), 160 * 1024, lds_allowed)) return OFQ_ERR_LAUNCH;
  kern<<<grid, NW * 64, lds, st>>>(g, m, k, group_size, ilog2_exact(group_size / 128),
                                  rows_per_block);
  return ofq_check_launch();
}

// the smallest common rows_per_block (>= 16, <= max_rows) whose blocks fit one resident round:
// 256 blocks of 16 waves, else 512 of 8; returns the grid size
int64_t grouped_split(const LinearArgs* pr, int count, int max_rows, int* rpb_out) {
  constexpr int kCUs = 256;
  int64_t n_total = 0;
  for (int i = 0; i < count; ++i) n_total += pr[i].n;
  auto blocks_at = [&](int rpb) {
    int64_t b = 0;
    for (int i = 0; i < count; ++i) b += (pr[i].n + rpb - 1) / rpb;
    return b;
  };
  int rpb = (int)((n_total + kCUs - 1) / kCUs);
  if (rpb < 16) rpb = 16;
  while (rpb < max_rows && blocks_at(rpb) > kCUs) ++rpb;
  if (rpb > max_rows || blocks_at(rpb) > kCUs) {
    rpb = (int)((n_total + 2 * kCUs - 1) / (2 * kCUs));
    if (rpb < 16) rpb = 16;
    while (rpb < max_rows && blocks_at(rpb) > 2 * kCUs) ++rpb;
  }
  if (rpb > max_rows) rpb = max_rows;
  *rpb_out = rpb;
  return blocks_at(rpb);
}

void fill_group(GemvGroup& g, const LinearArgs* pr, int count, int rpb) {
  g.count = count;
  int first = 0;
  for (int i = 0; i < count; ++i) {
    g.p[i].x = pr[i].x;
    g.p[i].w = static_cast<const uint8_t*>(pr[i].w);
    g.p[i].scale = pr[i].scale;
    g.p[i].zero = pr[i].zero;
    g.p[i].bias = pr[i].bias;
    g.p[i].out = pr[i].out;
    g.p[i].N = (int)pr[i].n;
    g.p[i].first_block = first;
    first += (int)((pr[i].n + rpb - 1) / rpb);
  }
}

// fp16, 4-bit codes, groups in multiples of 128: the kernel of the single-problem fast path
int launch_w4p_grouped(hipStream_t st, const LinearArgs* pr, int count) {
  const LinearArgs& a = pr[0];
  int rpb = 0;
  const int64_t grid = grouped_split(pr, count, 16 * kW4pMaxTiles, &rpb);
  if (grid > 0x7FFFFFFF) return OFQ_ERR_UNSUPPORTED;
  const bool two_per_cu = grid > 256;
  const int nw = two_per_cu ? 8 : 16;
  if ((int64_t)((rpb + 15) / 16) * a.m * 16 > nw * 64) return OFQ_ERR_UNSUPPORTED;
  const bool exact = !(a.symmetric && a.w_signed);
  const size_t lds_cap = (two_per_cu ? 80u : 160u) * 1024u;
  size_t lds = gemv_w4p_lds_bytes(nw, (int)a.m, (int)a.k, (int)a.group_size, rpb, exact,
                                  !a.symmetric);
  // x beyond one staging: two stagings, each of half the chunk pairs of a row
  const bool two_stagings = a.m * a.k / 16 > (int64_t)kGemvMaxUnits * nw * 64 || lds > lds_cap;
  if (two_stagings) {
    lds = gemv_w4p_lds_bytes(nw, (int)a.m, (int)a.k, (int)a.group_size, rpb, exact, !a.symmetric,
                             1, 2);
    const int64_t half_units = a.m * gemv_w4p_phase_chunks((int)a.k, 2) * 8;
    if (half_units > (int64_t)kGemvMaxUnits * nw * 64 || lds > lds_cap) return OFQ_ERR_UNSUPPORTED;
  }
  GemvGroup g{};
  fill_group(g, pr, count, rpb);
#define OFQ_W4PG(NWV, PHV)                                                                   \
  if (nw == NWV && two_stagings == (PHV == 2)) {                                             \
    if (!exact)                                                                              \
      return launch_w4p_grouped_inst<NWV, false, true, kZeroNone, PHV>(                      \
          st, g, (int)grid, (int)a.m, (int)a.k, (int)a.group_size, rpb, lds);                \
    if (a.symmetric)                                                                         \
      return launch_w4p_grouped_inst<NWV, true, false, kZeroSymU, PHV>(                      \
          st, g, (int)grid, (int)a.m, (int)a.k, (int)a.group_size, rpb, lds);                \
    return launch_w4p_grouped_inst<NWV, true, false, kZeroAsym, PHV>(                        \
        st, g, (int)grid, (int)a.m, (int)a.k, (int)a.group_size, rpb, lds);                  \
  }
  OFQ_W4PG(16, 1) OFQ_W4PG(8, 1) OFQ_W4PG(16, 2) OFQ_W4PG(8, 2)
#undef OFQ_W4PG
  return OFQ_ERR_UNSUPPORTED;
}

template<int NW, bool EXACT, bool SIGNED, int ZMODE, int PH = 1>
int launch_w4p_glu_inst(hipStream_t st, const LinearArgs& a, const GluArgs& glu, int grid,
                        int rows_per_block, size_t lds) {
  auto kern = gemv_w4p_f16_glu<NW, EXACT, SIGNED, ZMODE, PH>;
  static std::atomic<uint64_t> lds_allowed{0};  // devices on which the kernel's LDS limit is raised
  if (!ofq_allow_dynamic_lds(reinterpret_cast<const void*>(kern), 160 * 1024, lds_allowed)) return OFQ_ERR_LAUNCH;
  kern<<<grid, NW * 64, lds, st>>>(static_cast<const f16*>(a.x), static_cast<const uint8_t*>(a.w),
                                  static_cast<const f16*>(a.scale),
                                  static_cast<const f16*>(a.zero),
                                  static_cast<const f16*>(a.bias), static_cast<f16*>(a.out), glu,
                                  (int)a.m, (int)a.n, (int)a.k, (int)a.group_size,
                                  ilog2_exact(a.group_size / 128), rows_per_block);
  return ofq_check_launch();
}

}  // namespace

int launch_gemv_glu(hipStream_t st, const LinearArgs& a, const LinearArgs& g, void* y, int act) {
  {
    const int rc = launch_gemv_m1_glu(st, a, g, y, act);
    if (rc != OFQ_ERR_UNSUPPORTED) return rc;
  }
  if (!w4p_supported(a) || !w4p_supported(g)) return OFQ_ERR_UNSUPPORTED;
  if (g.n != a.n || g.k != a.k || g.m != a.m || g.x != a.x) return OFQ_ERR_UNSUPPORTED;
  constexpr int kCUs = 256;
  const bool exact = !(a.symmetric && a.w_signed);
  // A block walks the same rows of both weights.  First choice: up to 64 rows of each per block,
  // so that n = 11008 is one block of 16 waves per CU as in the plain linear (43 rows, three
  // tiles per weight); that doubles the per-(tile, wave) sums in LDS, so with many rows of x it
  // may not fit, and then a block owns at most 32 rows of each weight (two blocks per CU).
  int64_t grid = 0;
  int rpb = 0, nw = 0;
  size_t lds = 0;
  bool two_stagings = false, fits = false;
  for (int tiles_per_weight = kW4pMaxTiles; tiles_per_weight >= kW4pMaxTiles / 2 && !fits;
       tiles_per_weight -= kW4pMaxTiles / 2) {
    const int64_t max_rows = 16 * tiles_per_weight;
    grid = kCUs;
    if ((a.n + grid - 1) / grid > max_rows) grid = 2 * kCUs;
    if ((a.n + grid - 1) / grid > max_rows) grid = (a.n + max_rows - 1) / max_rows;
    rpb = (int)((a.n + grid - 1) / grid);
    if (rpb < 16) rpb = 16;
    grid = (a.n + rpb - 1) / rpb;
    const bool two_per_cu = grid > kCUs;
    nw = two_per_cu ? 8 : 16;
    // one thread folds one output of the block (per weight)
    if ((int64_t)((rpb + 15) / 16) * a.m * 16 > nw * 64) continue;
    const size_t lds_cap = (two_per_cu ? 80u : 160u) * 1024u;
    lds = gemv_w4p_lds_bytes(nw, (int)a.m, (int)a.k, (int)a.group_size, rpb, exact, !a.symmetric,
                             2);
    // x beyond one staging (8 rows of 4096 next to the sums of two weights): two stagings
    two_stagings = a.m * a.k / 16 > (int64_t)kGemvMaxUnits * nw * 64 || lds > lds_cap;
    if (two_stagings) {
      lds = gemv_w4p_lds_bytes(nw, (int)a.m, (int)a.k, (int)a.group_size, rpb, exact,
                               !a.symmetric, 2, 2);
      const int64_t half_units = a.m * gemv_w4p_phase_chunks((int)a.k, 2) * 8;
      if (half_units > (int64_t)kGemvMaxUnits * nw * 64 || lds > lds_cap) continue;
    }
    fits = true;
  }
  if (!fits) return OFQ_ERR_UNSUPPORTED;
  GluArgs glu;
  glu.w2 = static_cast<const uint8_t*>(g.w);
  glu.scale2 = static_cast<const f16*>(g.scale);
  glu.zero2 = static_cast<const f16*>(g.zero);
  glu.bias2 = static_cast<const f16*>(g.bias);
  glu.out2 = static_cast<f16*>(g.out);
  glu.y = static_cast<f16*>(y);
  glu.act = act;
#define OFQ_W4PGLU(NWV, PHV)                                                                   \
  if (nw == NWV && two_stagings == (PHV == 2)) {                                               \
    if (!exact)                                                                                \
      return launch_w4p_glu_inst<NWV, false, true, kZeroNone, PHV>(st, a, glu, (int)grid, rpb, \
                                                                   lds);                       \
    if (a.symmetric)                                                                           \
      return launch_w4p_glu_inst<NWV, true, false, kZeroSymU, PHV>(st, a, glu, (int)grid, rpb, \
                                                                   lds);                       \
    return launch_w4p_glu_inst<NWV, true, false, kZeroAsym, PHV>(st, a, glu, (int)grid, rpb,   \
                                                                 lds);                         \
  }
  OFQ_W4PGLU(16, 1) OFQ_W4PGLU(8, 1) OFQ_W4PGLU(16, 2) OFQ_W4PGLU(8, 2)
#undef OFQ_W4PGLU
  return OFQ_ERR_UNSUPPORTED;
}

int launch_gemv_grouped(hipStream_t st, const LinearArgs* pr, int count) {
  if (count < 1 || count > kGemvMaxProblems) return OFQ_ERR_UNSUPPORTED;
  {
    const int rc = launch_gemv_m1_grouped(st, pr, count);
    if (rc != OFQ_ERR_UNSUPPORTED) return rc;
  }
  const LinearArgs& a = pr[0];
  bool all_w4p = true;
  for (int i = 0; i < count; ++i) {
    const LinearArgs& b = pr[i];
    if (!rows_supported(b)) return OFQ_ERR_UNSUPPORTED;
    if (b.t_dtype != a.t_dtype || b.bits != a.bits || b.w_signed != a.w_signed
        || b.symmetric != a.symmetric || b.group_size != a.group_size || b.m != a.m
        || b.k != a.k) {
      return OFQ_ERR_UNSUPPORTED;
    }
    all_w4p = all_w4p && w4p_supported(b);
  }
  if (all_w4p) {
    const int rc = launch_w4p_grouped(st, pr, count);
    if (rc != OFQ_ERR_UNSUPPORTED) return rc;
  }
  int rpb = 0;
  const int64_t grid = grouped_split(pr, count, 16 * kRowsMaxTiles, &rpb);
  if (grid > 0x7FFFFFFF) return OFQ_ERR_UNSUPPORTED;
  const bool two_per_cu = grid > 256;
  const int nw = two_per_cu ? 8 : 16;
  const size_t cap = (two_per_cu ? 80u : 160u) * 1024u;
  bool staged = a.m * a.k / 8 <= (int64_t)kRowsMaxUnits * nw * 64;
  size_t lds = gemv_rows_lds_bytes(nw, (int)a.m, (int)a.k, (int)a.group_size, rpb, !a.symmetric,
                                   staged);
  if (staged && lds > cap) {
    staged = false;
    lds = gemv_rows_lds_bytes(nw, (int)a.m, (int)a.k, (int)a.group_size, rpb, !a.symmetric,
                              false);
  }
  if (lds > cap) return OFQ_ERR_UNSUPPORTED;
  GemvGroup g{};
  fill_group(g, pr, count, rpb);
#define OFQ_RG(TT_, NWV)                                                                   \
  return staged ? launch_rows_grouped_t<TT_, NWV, true>(st, a, g, (int)grid, rpb, lds)     \
                : launch_rows_grouped_t<TT_, NWV, false>(st, a, g, (int)grid, rpb, lds)
  if (a.t_dtype == OFQ_BF16) {
    if (nw == 16) { OFQ_RG(bf16, 16); }
    OFQ_RG(bf16, 8);
  }
  if (nw == 16) { OFQ_RG(f16, 16); }
  OFQ_RG(f16, 8);
#undef OFQ_RG
}

bool gemv_mt_supported(const LinearArgs& a) {
  // beyond 64 rows the weights would be walked twice and the tiled GEMM with K slices is faster
  if (a.m <= 16 || a.m > 64) return false;
  LinearArgs b = a;
  b.m = 16;  // the same shape rules as the decode kernel
  return rows_supported(b) && a.n * a.k <= 0x7FFFFFFFLL * 8;
}

int launch_gemv_mt(hipStream_t st, const LinearArgs& a) {
  for (int64_t m0 = 0; m0 < a.m; m0 += 64) {
    const int m = (int)(a.m - m0 < 64 ? a.m - m0 : 64);
    const int rc = launch_rows_mt_part(st, a, m0, m);
    if (rc != OFQ_OK) return rc;  // OFQ_ERR_UNSUPPORTED can only come from the first part
  }
  return OFQ_OK;
}

bool gemv_wq_supported(const LinearArgs& a) {
  if (rows_supported(a)) return true;
  if (a.t_dtype != OFQ_F16 || a.group_dim != 1 || a.m > 16 || a.m < 1) return false;
  const int ch = a.bits == 4 ? 128 : 64;
  const int lk = ch / 4;
  if (a.k % ch != 0 || a.group_size % lk != 0) return false;
  if (a.n * a.k > 0x7FFFFFFFLL * 8 || a.k > 0x7FFFFFFF || a.n > 0x7FFFFFFF - 16) return false;
  return true;
}

int launch_gemv_wq(hipStream_t st, const LinearArgs& a) {
  if (gemv_m1_supported(a)) {
    const int rc = launch_gemv_m1(st, a);
    if (rc != OFQ_ERR_UNSUPPORTED) return rc;
  }
  if (gemv_m1_any_supported(a)) {
    const int rc = launch_gemv_m1_any(st, a);
    if (rc != OFQ_ERR_UNSUPPORTED) return rc;
  }
  if (w4s_supported(a)) {
    const int rc = launch_w4s(st, a);
    if (rc != OFQ_ERR_UNSUPPORTED) return rc;
  } else if (w4p_supported(a)) {
    // uint8 container / asymmetric: the row-balanced kernel with the reference's roundings
    const int rc = launch_w4p(st, a, ilog2_exact(a.group_size / 128), false);
    if (rc != OFQ_ERR_UNSUPPORTED) return rc;
  }
  if (rows_supported(a)) {
    const int rc = launch_rows(st, a);
    if (rc != OFQ_ERR_UNSUPPORTED) return rc;
  }
  if (a.t_dtype != OFQ_F16) return OFQ_ERR_UNSUPPORTED;  // the kernels below are fp16 only
  {
    const int ch = a.bits == 4 ? 128 : 64;
    if (a.k % ch != 0 || a.group_size % (ch / 4) != 0) return OFQ_ERR_UNSUPPORTED;
  }
  const int zmode = !a.symmetric ? kZeroAsym : (a.w_signed ? kZeroNone : kZeroSymU);
#define OFQ_V(B, SG, ZM) \
  if (a.bits == B && a.w_signed == SG && zmode == ZM) return launch_gemv_variant<B, SG, ZM>(st, a);
  OFQ_V(4, true, kZeroNone)
  OFQ_V(4, false, kZeroSymU)
  OFQ_V(4, false, kZeroAsym)
  OFQ_V(8, true, kZeroNone)
  OFQ_V(8, false, kZeroSymU)
  OFQ_V(8, false, kZeroAsym)
#undef OFQ_V
  return OFQ_ERR_UNSUPPORTED;
}

int launch_linear_generic(hipStream_t st, const LinearArgs& a) {
  if (rows_f32_supported(a)) {
    const int rc = launch_rows_f32(st, a);
    if (rc != OFQ_ERR_UNSUPPORTED) return rc;
  }
  if (a.m > 65535) return OFQ_ERR_UNSUPPORTED;
  switch (a.t_dtype) {
    case OFQ_F16: return launch_generic_t<f16>(st, a);
    case OFQ_BF16: return launch_generic_t<bf16>(st, a);
    case OFQ_F32: return launch_generic_t<float>(st, a);
    default: return OFQ_ERR_BAD_DTYPE;
  }
}

}  // namespace ofq

using namespace ofq;

extern "C" size_t ofq_fused_linear_gq_workspace_bytes(int w_dtype, int t_dtype, int num_bits,
                                                      int symmetric, int group_dim,
                                                      int64_t group_size, int64_t m, int64_t n,
                                                      int64_t k) {
  if ((num_bits != 4 && num_bits != 8) || group_size <= 0 || m <= 0 || n <= 0 || k <= 0) return 0;
  LinearArgs a{};
  a.t_dtype = t_dtype;
  a.w_signed = w_dtype == OFQ_I8;
  a.bits = num_bits;
  a.symmetric = symmetric != 0;
  a.group_dim = group_dim;
  a.group_size = group_size;
  a.m = m;
  a.n = n;
  a.k = k;
  if (gemv_wq_supported(a) || gemv_m1_any_supported(a) || gemv_mt_supported(a)) return 0;
  if (group_dim == 0) return gemm_gn_workspace_bytes(a);
  return gemm_wq_workspace_bytes(a);  // 0 for every path but the two-pass GEMM at large m
}

extern "C" int ofq_fused_linear_gq(void* stream, const void* x, const void* w,
                                   const void* w_scale, const void* w_zero, const void* b,
                                   void* out, int w_dtype, int t_dtype, int num_bits,
                                   int symmetric, int group_dim, int64_t group_size, int64_t m,
                                   int64_t n, int64_t k, void* workspace, size_t workspace_bytes) {
  // checks of FusedLinearWithGroupwiseQuantizedWeightKernel::Compute,
  // groupwise_quantization_kernels.cu:773-822
  OFQ_RETURN_IF(num_bits != 4 && num_bits != 8, OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(group_dim != 0 && group_dim != 1, OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(w_dtype != OFQ_U8 && w_dtype != OFQ_I8, OFQ_ERR_BAD_DTYPE);
  OFQ_RETURN_IF(!symmetric && w_dtype != OFQ_U8, OFQ_ERR_BAD_DTYPE);
  OFQ_RETURN_IF(t_dtype != OFQ_F16 && t_dtype != OFQ_BF16 && t_dtype != OFQ_F32,
                OFQ_ERR_BAD_DTYPE);
  OFQ_RETURN_IF(m < 0 || n < 0 || k <= 0, OFQ_ERR_BAD_SHAPE);
  OFQ_RETURN_IF(k % (8 / num_bits) != 0, OFQ_ERR_BAD_SHAPE);
  const int64_t group_dim_size = group_dim == 0 ? n : k;
  OFQ_RETURN_IF(group_size <= 0, OFQ_ERR_BAD_ATTR);
  if (m == 0 || n == 0) return OFQ_OK;
  OFQ_RETURN_IF(group_size > group_dim_size || group_dim_size % group_size != 0,
                OFQ_ERR_BAD_SHAPE);
  // int32 index limits of the reference launchers, :651-655
  const int64_t i32max = 0x7FFFFFFF;
  OFQ_RETURN_IF(m * k > i32max || n * k > i32max || m * n > i32max, OFQ_ERR_UNSUPPORTED);
  OFQ_RETURN_IF(x == nullptr || w == nullptr || w_scale == nullptr || out == nullptr,
                OFQ_ERR_NULL_POINTER);
  OFQ_RETURN_IF((symmetric != 0) != (w_zero == nullptr), OFQ_ERR_NULL_POINTER);
  OFQ_RETURN_IF(!ofq_aligned16(x) || !ofq_aligned16(w) || !ofq_aligned16(w_scale)
                    || !ofq_aligned16(w_zero) || !ofq_aligned16(b) || !ofq_aligned16(out),
                OFQ_ERR_MISALIGNED);
  LinearArgs a;
  a.x = x;
  a.w = w;
  a.scale = w_scale;
  a.zero = w_zero;
  a.bias = b;
  a.out = out;
  a.t_dtype = t_dtype;
  a.w_signed = w_dtype == OFQ_I8;
  a.bits = num_bits;
  a.symmetric = symmetric != 0;
  a.group_dim = group_dim;
  a.group_size = group_size;
  a.m = m;
  a.n = n;
  a.k = k;
  hipStream_t st = static_cast<hipStream_t>(stream);
  // (the row-per-wave kernel for one row of x covers rows and groups off the chunk grid of the
  // MFMA kernels: k a multiple of 32 / 16 elements, groups from 32 / 16)
  if (gemv_wq_supported(a) || gemv_m1_any_supported(a)) {
    const int rc = launch_gemv_wq(st, a);
    if (rc != OFQ_ERR_UNSUPPORTED) return rc;  // e.g. bf16 with an x too large to stage
  }
  if (gemv_mt_supported(a)) {
    const int rc = launch_gemv_mt(st, a);
    if (rc != OFQ_ERR_UNSUPPORTED) return rc;
  }
  if (gemm_wq_supported(a)) return launch_gemm_wq(st, a, workspace, workspace_bytes);
  if (a.group_dim == 0) {
    const size_t need = gemm_gn_workspace_bytes(a);
    if (need != 0 && workspace != nullptr && workspace_bytes >= need && ofq_aligned16(workspace)) {
      return launch_gemm_gn(st, a, workspace);
    }
    if (gemv_gn_supported(a)) {
      const int rc = launch_gemv_gn(st, a);
      if (rc != OFQ_ERR_UNSUPPORTED) return rc;
    }
  }
  return launch_linear_generic(st, a);
}

// ---- tile-major weight copy -------------------------------------------------------------------
namespace ofq {
namespace {

// one lane moves the 16 bytes it will later request: lane (k-slot kb, row r) of chunk c of tile t
// of block b <- row b * rows_per_block + 16 t + r, bytes [64 c + 16 kb, +16); rows past the
// block's share (or past n) become zeros
__global__ void __launch_bounds__(256)
repack_w4_tiles(const uint8_t* __restrict__ w, uint8_t* __restrict__ tiled, int N, int K,
                int rows_per_block, int tiles_per_block, int64_t pieces) {
  const int nchunks = K >> 7;
  const int row_bytes = K >> 1;
  for (int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x; p < pieces;
       p += (int64_t)gridDim.x * 256) {
    const int lane = (int)(p & 63);
    const int64_t kb_index = p >> 6;  // (block * tiles_per_block + t) * nchunks + c
    const int c = (int)(kb_index % nchunks);
    const int64_t tile_index = kb_index / nchunks;
    const int t = (int)(tile_index % tiles_per_block);
    const int64_t b = tile_index / tiles_per_block;
    const int r = lane & 15, kb = lane >> 4;
    const int row_l = 16 * t + r;
    const int64_t row = b * rows_per_block + row_l;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (row_l < rows_per_block && row < N) {
      v = *reinterpret_cast<const u32x4*>(w + row * row_bytes + c * 64 + kb * 16);
    }
    reinterpret_cast<u32x4*>(tiled)[p] = v;
  }
}

bool tiled_shape_ok(int num_bits, int64_t n, int64_t k) {
  return num_bits == 4 && n >= 1 && k >= 128 && k % 128 == 0 && k <= (1 << 20)
         && n <= 0x7FFFFFFF - 16;
}

}  // namespace
}  // namespace ofq

extern "C" size_t ofq_groupwise_repack_bytes(int num_bits, int64_t n, int64_t k) {
  if (!tiled_shape_ok(num_bits, n, k)) return 0;
  int64_t grid;
  int rpb;
  w4p_row_split(n, &grid, &rpb);
  return (size_t)grid * (size_t)((rpb + 15) / 16) * 16 * (size_t)(k / 2);
}

extern "C" int ofq_groupwise_repack(void* stream, const void* w, void* w_tiled, int num_bits,
                                    int64_t n, int64_t k) {
  OFQ_RETURN_IF(num_bits != 4 && num_bits != 8, OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(n <= 0 || k <= 0, OFQ_ERR_BAD_SHAPE);
  OFQ_RETURN_IF(!tiled_shape_ok(num_bits, n, k), OFQ_ERR_UNSUPPORTED);
  OFQ_RETURN_IF(w == nullptr || w_tiled == nullptr, OFQ_ERR_NULL_POINTER);
  OFQ_RETURN_IF(!ofq_aligned16(w) || !ofq_aligned16(w_tiled), OFQ_ERR_MISALIGNED);
  int64_t grid;
  int rpb;
  w4p_row_split(n, &grid, &rpb);
  const int tpb = (rpb + 15) / 16;
  const int64_t pieces = grid * tpb * (k / 128) * 64;
  int64_t blocks = (pieces + 255) / 256;
  if (blocks > 256 * 64) blocks = 256 * 64;
  repack_w4_tiles<<<(unsigned)blocks, 256, 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const uint8_t*>(w), static_cast<uint8_t*>(w_tiled), (int)n, (int)k, rpb, tpb,
      pieces);
  return ofq_check_launch();
}

extern "C" int ofq_fused_linear_gq_tiled(void* stream, const void* x, const void* w_tiled,
                                         const void* w_scale, const void* w_zero, const void* b,
                                         void* out, int w_dtype, int t_dtype, int num_bits,
                                         int symmetric, int group_dim, int64_t group_size,
                                         int64_t m, int64_t n, int64_t k) {
  OFQ_RETURN_IF(num_bits != 4 && num_bits != 8, OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(group_dim != 0 && group_dim != 1, OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(w_dtype != OFQ_U8 && w_dtype != OFQ_I8, OFQ_ERR_BAD_DTYPE);
  OFQ_RETURN_IF(!symmetric && w_dtype != OFQ_U8, OFQ_ERR_BAD_DTYPE);
  OFQ_RETURN_IF(t_dtype != OFQ_F16 && t_dtype != OFQ_BF16 && t_dtype != OFQ_F32,
                OFQ_ERR_BAD_DTYPE);
  OFQ_RETURN_IF(m < 0 || n < 0 || k <= 0 || group_size <= 0, OFQ_ERR_BAD_SHAPE);
  if (m == 0 || n == 0) return OFQ_OK;
  const int64_t group_dim_size = group_dim == 0 ? n : k;
  OFQ_RETURN_IF(group_size > group_dim_size || group_dim_size % group_size != 0,
                OFQ_ERR_BAD_SHAPE);
  OFQ_RETURN_IF(x == nullptr || w_tiled == nullptr || w_scale == nullptr || out == nullptr,
                OFQ_ERR_NULL_POINTER);
  OFQ_RETURN_IF((symmetric != 0) != (w_zero == nullptr), OFQ_ERR_NULL_POINTER);
  OFQ_RETURN_IF(!ofq_aligned16(x) || !ofq_aligned16(w_tiled) || !ofq_aligned16(w_scale)
                    || !ofq_aligned16(w_zero) || !ofq_aligned16(b) || !ofq_aligned16(out),
                OFQ_ERR_MISALIGNED);
  LinearArgs a;
  a.x = x;
  a.w = w_tiled;
  a.scale = w_scale;
  a.zero = w_zero;
  a.bias = b;
  a.out = out;
  a.t_dtype = t_dtype;
  a.w_signed = w_dtype == OFQ_I8;
  a.bits = num_bits;
  a.symmetric = symmetric != 0;
  a.group_dim = group_dim;
  a.group_size = group_size;
  a.m = m;
  a.n = n;
  a.k = k;
  // what the row-balanced kernel takes: fp16, 4 bits, groups of a multiple of 128 along K, at
  // most 16 rows of x whose m * k halves fit LDS
  if (!w4p_supported(a) || !tiled_shape_ok(num_bits, n, k)) return OFQ_ERR_UNSUPPORTED;
  return launch_w4p(static_cast<hipStream_t>(stream), a, ilog2_exact(a.group_size / 128), true);
}
