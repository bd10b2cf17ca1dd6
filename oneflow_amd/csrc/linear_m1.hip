// Launchers of the decode kernels for a single row of x (gemv_w4_m1.h): a wave owns whole weight
// rows.  fp16, 4-bit symmetric codes in an int8 container, groups along K.
#include "gemv_w4_m1.h"
#include "ofq_device.h"
#include "ofq_internal.h"

namespace ofq {
namespace {

inline int log2_exact(int64_t v) {
  if (v <= 0 || (v & (v - 1)) != 0) return -1;
  int s = 0;
  while ((1LL << s) < v) ++s;
  return s;
}

template<int NW, int H, int XU>
int launch_m1_inst(hipStream_t st, const LinearArgs& a) {
  M1Shape sh;
  sh.N = (int)a.n;
  sh.K = (int)a.k;
  sh.rows_per_block = NW;  // one row per wave
  sh.gshift = log2_exact(a.group_size);
  sh.G = (int)(a.k / a.group_size);
  const int grid = (int)((a.n + NW - 1) / NW);
  gemv_w4_m1<NW, 1, H, XU><<<grid, NW * 64, gemv_m1_lds_bytes(H), st>>>(
      static_cast<const f16*>(a.x), static_cast<const uint8_t*>(a.w),
      static_cast<const f16*>(a.scale), static_cast<const f16*>(a.bias), static_cast<f16*>(a.out),
      sh);
  return ofq_check_launch();
}

}  // namespace

bool gemv_m1_supported(const LinearArgs& a) {
  return a.m == 1 && a.t_dtype == OFQ_F16 && a.bits == 4 && a.w_signed && a.symmetric
         && a.group_dim == 1 && a.group_size >= 128 && log2_exact(a.group_size) >= 0
         && a.k % 256 == 0 && a.k <= 16384 && a.k % a.group_size == 0 && a.n >= 1
         && a.n <= (1 << 24);
}

// Blocks of 16 waves when a row is at most 2 KB of codes (k <= 4096), of 8 waves beyond: with
// longer rows two small blocks per CU, each with its own barrier, run ahead of one large one
// (4096 x 11008: 6.3 against 6.7 us), with short rows the second staging of x costs more than
// that gains (4096 x 4096: 3.55 against 3.8 us).
int launch_gemv_m1(hipStream_t st, const LinearArgs& a) {
  const int h = (int)((a.k / 2 + 1023) / 1024);
  if (a.k <= 4096) {
    switch (h) {
      case 1: return launch_m1_inst<16, 1, 1>(st, a);
      default: return launch_m1_inst<16, 2, 1>(st, a);
    }
  }
  switch (h) {
    case 3: return launch_m1_inst<8, 3, 1>(st, a);
    case 4: return launch_m1_inst<8, 4, 1>(st, a);
    case 5: return launch_m1_inst<8, 5, 2>(st, a);
    case 6: return launch_m1_inst<8, 6, 2>(st, a);
    case 7: return launch_m1_inst<8, 7, 2>(st, a);
    case 8: return launch_m1_inst<8, 8, 2>(st, a);
    default: return OFQ_ERR_UNSUPPORTED;
  }
}

}  // namespace ofq
