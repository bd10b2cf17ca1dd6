// fused_linear_with_groupwise_quantized_weight, groups along N (group_dim = 0): launchers of the
// streaming kernels of gemv_rows_gn.h (fp16 / bf16, and fp32 with 16 rows of x per pass).  x is taken 64 rows at a time (each pass
// streams the weights once), so any m runs; at large m the caller prefers the two-pass GEMM when
// it has a workspace.
#include <atomic>
#include "gemv_rows_gn.h"
#include "ofq_device.h"
#include "ofq_internal.h"

namespace ofq {
namespace {

template<typename T, int BITS, bool SIGNED, int ZMODE, int NW, int MT, bool XLDS>
int launch_gn_inst(hipStream_t st, const LinearArgs& a, const void* x, void* out, int m, int grid,
                   int rows_per_block, size_t lds) {
  auto kern = gemv_rows_gn<T, BITS, SIGNED, ZMODE, NW, MT, XLDS>;
  static std::atomic<uint64_t> lds_allowed{0};  // devices on which the kernel's LDS limit is raised
  if (!ofq_allow_dynamic_lds(reinterpret_cast<const void*>(kern), 160 * 1024, lds_allowed)) return OFQ_ERR_LAUNCH;
  kern<<<grid, NW * 64, lds, st>>>(
      static_cast<const uint16_t*>(x), static_cast<const uint8_t*>(a.w),
      static_cast<const uint16_t*>(a.scale), static_cast<const uint16_t*>(a.zero),
      static_cast<const uint16_t*>(a.bias), static_cast<uint16_t*>(out), m, (int)a.n, (int)a.k,
      (int)a.group_size, rows_per_block);
  return ofq_check_launch();
}

template<typename T, int NW, int MT, bool XLDS>
int launch_gn_t(hipStream_t st, const LinearArgs& a, const void* x, void* out, int m, int grid,
                int rpb, size_t lds) {
  const int zmode = !a.symmetric ? kZeroAsym : (a.w_signed ? kZeroNone : kZeroSymU);
#define OFQ_R(B, SG, ZM)                              \
  if (a.bits == B && a.w_signed == SG && zmode == ZM) \
    return launch_gn_inst<T, B, SG, ZM, NW, MT, XLDS>(st, a, x, out, m, grid, rpb, lds);
  OFQ_R(4, true, kZeroNone)
  OFQ_R(4, false, kZeroSymU)
  OFQ_R(4, false, kZeroAsym)
  OFQ_R(8, true, kZeroNone)
  OFQ_R(8, false, kZeroSymU)
  OFQ_R(8, false, kZeroAsym)
#undef OFQ_R
  return OFQ_ERR_UNSUPPORTED;
}

// tiles of x per pass (1, 2 or 4) and the waves that go with them
inline int gn_mt(int m) { return m <= 16 ? 1 : (m <= 32 ? 2 : 4); }
inline int gn_waves(int mt) { return mt == 4 ? 12 : 16; }

// Rows per block: whole 16-row tiles, about one block per CU, at most kRowsMaxTiles tiles, and
// few enough that the scale rows of the groups a block touches fit in LDS beside the sums.
int gn_rows_per_block(const LinearArgs& a, int mt) {
  constexpr int kCUs = 256;
  int rpb = (int)(((a.n + kCUs - 1) / kCUs + 15) / 16 * 16);
  if (rpb > 16 * kRowsMaxTiles) rpb = 16 * kRowsMaxTiles;
  if (rpb < 16) rpb = 16;
  while (rpb > 16
         && gemv_rows_gn_lds_bytes(gn_waves(mt), mt, (int)a.k, (int)a.group_size, rpb,
                                   !a.symmetric)
                > 160u * 1024u) {
    rpb -= 16;
  }
  return rpb;
}

int launch_gn_part(hipStream_t st, const LinearArgs& a, int64_t m0, int m) {
  const int mt = gn_mt(m);
  const int nw = gn_waves(mt);
  const int rpb = gn_rows_per_block(a, mt);
  // 33 to 64 rows of x whose buffers do not fit beside the scale rows: two passes of up to 32
  // rows with buffers are faster than one pass with x straight from L2 when the rows are long
  // (4096 x 11008 with a zero point, 64 rows: 60 us in one pass, 37 in two; with k = 4096 the
  // two are level in fp16 and one pass is ahead in bf16)
  if (mt == 4) {
    const size_t lds4 = gemv_rows_gn_lds_bytes(8, 4, (int)a.k, (int)a.group_size, rpb,
                                               !a.symmetric, a.bits, true);
    const int rpb2 = gn_rows_per_block(a, 2);
    const size_t lds2 = gemv_rows_gn_lds_bytes(12, 2, (int)a.k, (int)a.group_size, rpb2,
                                               !a.symmetric, a.bits, true);
    if (a.k >= 8192 && lds4 > 160u * 1024u && lds2 <= 160u * 1024u) {
      const int rc = launch_gn_part(st, a, m0, 32);
      if (rc != OFQ_OK) return rc;
      return launch_gn_part(st, a, m0 + 32, m - 32);
    }
  }
  const int grid = (int)((a.n + rpb - 1) / rpb);
  const void* x = static_cast<const char*>(a.x) + (size_t)m0 * a.k * 2;
  void* out = static_cast<char*>(a.out) + (size_t)m0 * a.n * 2;
  // More than 16 rows of x: x through per-wave buffers in LDS when they fit beside the block's
  // scale rows (12 / 8 waves for two / four tiles of x).  Up to 16 rows the direct requests
  // touch few enough cache lines (11008 x 4096, fp16 with a zero point, 2 rows: 10.8 us direct,
  // 12.1 us through the buffers; 32 rows: 19.5 against 15.0).
  if (mt > 1) {
    const int nwx = mt == 2 ? 12 : 8;
    const size_t ldsx = gemv_rows_gn_lds_bytes(nwx, mt, (int)a.k, (int)a.group_size, rpb,
                                               !a.symmetric, a.bits, true);
    if (ldsx <= 160u * 1024u) {
#define OFQ_MTX(TT_)                                                                       \
  switch (mt) {                                                                            \
    case 2: return launch_gn_t<TT_, 12, 2, true>(st, a, x, out, m, grid, rpb, ldsx);       \
    default: return launch_gn_t<TT_, 8, 4, true>(st, a, x, out, m, grid, rpb, ldsx);       \
  }
      if (a.t_dtype == OFQ_BF16) { OFQ_MTX(bf16) }
      OFQ_MTX(f16)
#undef OFQ_MTX
    }
  }
  const size_t lds =
      gemv_rows_gn_lds_bytes(nw, mt, (int)a.k, (int)a.group_size, rpb, !a.symmetric);
  if (lds > 160u * 1024u) return OFQ_ERR_UNSUPPORTED;
#define OFQ_MT(TT_)                                                                          \
  switch (mt) {                                                                              \
    case 1: return launch_gn_t<TT_, 16, 1, false>(st, a, x, out, m, grid, rpb, lds);         \
    case 2: return launch_gn_t<TT_, 16, 2, false>(st, a, x, out, m, grid, rpb, lds);         \
    default: return launch_gn_t<TT_, 12, 4, false>(st, a, x, out, m, grid, rpb, lds);        \
  }
  if (a.t_dtype == OFQ_BF16) { OFQ_MT(bf16) }
  OFQ_MT(f16)
#undef OFQ_MT
}

// ---- fp32 activations: 16 rows of x per pass -------------------------------------------------------
template<int BITS, bool SIGNED, int ZMODE>
int launch_gn_f32_inst(hipStream_t st, const LinearArgs& a, const float* x, float* out, int m,
                       int grid, int rows_per_block, size_t lds) {
  auto kern = gemv_rows_f32_gn<BITS, SIGNED, ZMODE, 16>;
  static std::atomic<uint64_t> lds_allowed{0};  // devices on which the kernel's LDS limit is raised
  if (!ofq_allow_dynamic_lds(reinterpret_cast<const void*>(kern), 160 * 1024, lds_allowed)) return OFQ_ERR_LAUNCH;
  kern<<<grid, 16 * 64, lds, st>>>(x, static_cast<const uint8_t*>(a.w),
                                  static_cast<const float*>(a.scale),
                                  static_cast<const float*>(a.zero),
                                  static_cast<const float*>(a.bias), out, m, (int)a.n, (int)a.k,
                                  (int)a.group_size, rows_per_block);
  return ofq_check_launch();
}

int launch_gn_f32(hipStream_t st, const LinearArgs& a) {
  constexpr int kCUs = 256;
  int rpb = (int)(((a.n + kCUs - 1) / kCUs + 15) / 16 * 16);
  if (rpb > 16 * kRowsMaxTiles) rpb = 16 * kRowsMaxTiles;
  if (rpb < 16) rpb = 16;
  while (rpb > 16
         && gemv_rows_f32_gn_lds_bytes(16, (int)a.k, (int)a.group_size, rpb, !a.symmetric)
                > 160u * 1024u) {
    rpb -= 16;
  }
  const size_t lds = gemv_rows_f32_gn_lds_bytes(16, (int)a.k, (int)a.group_size, rpb, !a.symmetric);
  if (lds > 160u * 1024u) return OFQ_ERR_UNSUPPORTED;
  const int grid = (int)((a.n + rpb - 1) / rpb);
  const int zmode = !a.symmetric ? kZeroAsym : (a.w_signed ? kZeroNone : kZeroSymU);
  for (int64_t m0 = 0; m0 < a.m; m0 += 16) {
    const int m = (int)(a.m - m0 < 16 ? a.m - m0 : 16);
    const float* x = static_cast<const float*>(a.x) + m0 * a.k;
    float* out = static_cast<float*>(a.out) + m0 * a.n;
    int rc = OFQ_ERR_UNSUPPORTED;
#define OFQ_R(B, SG, ZM)                              \
  if (a.bits == B && a.w_signed == SG && zmode == ZM) \
    rc = launch_gn_f32_inst<B, SG, ZM>(st, a, x, out, m, grid, rpb, lds);
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

}  // namespace

bool gemv_gn_supported(const LinearArgs& a) {
  if (a.group_dim != 0) return false;
  if (a.t_dtype == OFQ_F32) {
    const int ck32 = a.bits == 4 ? 128 : 64;
    return (a.bits == 4 || a.bits == 8) && a.m >= 1 && a.k % ck32 == 0 && a.group_size % 16 == 0
           && a.n % a.group_size == 0 && (a.symmetric || !a.w_signed) && a.k <= (1 << 20)
           && a.n <= 0x7FFFFFFF - 64
           && gemv_rows_f32_gn_lds_bytes(16, (int)a.k, (int)a.group_size, 16, !a.symmetric)
                  <= 160u * 1024u;
  }
  if (a.t_dtype != OFQ_F16 && a.t_dtype != OFQ_BF16) return false;
  if ((a.bits != 4 && a.bits != 8) || a.m < 1) return false;
  const int ck = a.bits == 4 ? 128 : 64;
  if (a.k % ck != 0 || a.group_size % 16 != 0 || a.n % a.group_size != 0) return false;
  if (!a.symmetric && a.w_signed) return false;
  if (a.k > (1 << 20) || a.n > 0x7FFFFFFF - 64) return false;
  // the scale rows of one 16-row block must fit in LDS in the widest configuration
  return gemv_rows_gn_lds_bytes(16, 4, (int)a.k, (int)a.group_size, 16, !a.symmetric)
         <= 160u * 1024u;
}

int launch_gemv_gn(hipStream_t st, const LinearArgs& a) {
  if (a.t_dtype == OFQ_F32) return launch_gn_f32(st, a);
  if (gemv_m1_gn_supported(a)) {
    const int rc = launch_gemv_m1_gn(st, a);
    if (rc != OFQ_ERR_UNSUPPORTED) return rc;
  }
  for (int64_t m0 = 0; m0 < a.m; m0 += 64) {
    const int m = (int)(a.m - m0 < 64 ? a.m - m0 : 64);
    const int rc = launch_gn_part(st, a, m0, m);
    if (rc != OFQ_OK) return rc;  // OFQ_ERR_UNSUPPORTED can only come from the first part
  }
  return OFQ_OK;
}

}  // namespace ofq
