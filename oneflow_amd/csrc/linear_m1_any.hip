// Launcher of the single-row decode kernel for every 16-bit element type, code width, container
// and scheme (gemv_m1_any.h).  The fp16 / 4-bit / signed / symmetric case has a kernel of its
// own (linear_m1.hip) and is not instantiated here.
#include "gemv_m1_any.h"
#include "ofq_device.h"
#include "ofq_internal.h"

namespace ofq {
namespace {

inline int log2_pow2(int64_t v) {
  if (v <= 0 || (v & (v - 1)) != 0) return -1;
  int s = 0;
  while ((1LL << s) < v) ++s;
  return s;
}

// Blocks of 16 waves when a row is at most 2 KB of codes, of 8 waves beyond (two blocks per CU,
// each with its own barrier).  One row per wave while one resident round of blocks covers n;
// beyond that a block owns n / (resident blocks) consecutive rows, twice as many blocks from 128
// rows per block on.
template<typename T, int BITS, bool SIGNED, int ZMODE, int NW, int H>
int launch_any_inst(hipStream_t st, const LinearArgs& a) {
  constexpr int kCUs = 256;
  constexpr int slots = kCUs * (16 / NW);
  int64_t rpb = NW, grid = (a.n + NW - 1) / NW;
  if (grid > slots) {
    grid = slots;
    if ((a.n + grid - 1) / grid >= 128) grid *= 2;
    rpb = (a.n + grid - 1) / grid;
    grid = (a.n + rpb - 1) / rpb;
  }
  M1Shape sh;
  sh.N = (int)a.n;
  sh.K = (int)a.k;
  sh.rows_per_block = (int)rpb;
  sh.gshift = log2_pow2(a.group_size);
  sh.G = (int)(a.k / a.group_size);
  sh.gn = 1;
  gemv_m1_any<T, BITS, SIGNED, ZMODE, NW, H>
      <<<(int)grid, NW * 64, gemv_m1_any_lds_bytes<BITS>(H), st>>>(
          static_cast<const uint16_t*>(a.x), static_cast<const uint8_t*>(a.w),
          static_cast<const uint16_t*>(a.scale), static_cast<const uint16_t*>(a.zero),
          static_cast<const uint16_t*>(a.bias), static_cast<uint16_t*>(a.out), sh);
  return ofq_check_launch();
}

template<typename T, int BITS, bool SIGNED, int ZMODE>
int launch_any_h(hipStream_t st, const LinearArgs& a) {
  const int64_t row_bytes = a.k * BITS / 8;
  const int h = (int)((row_bytes + 1023) / 1024);
  switch (h) {
    case 1: return launch_any_inst<T, BITS, SIGNED, ZMODE, 16, 1>(st, a);
    case 2: return launch_any_inst<T, BITS, SIGNED, ZMODE, 16, 2>(st, a);
    case 3: return launch_any_inst<T, BITS, SIGNED, ZMODE, 8, 3>(st, a);
    case 4: return launch_any_inst<T, BITS, SIGNED, ZMODE, 8, 4>(st, a);
    default: return OFQ_ERR_UNSUPPORTED;
  }
}

template<typename T, int BITS>
int launch_any_scheme(hipStream_t st, const LinearArgs& a) {
  if (!a.symmetric) {
    return a.w_signed ? launch_any_h<T, BITS, true, kZeroAsym>(st, a)
                      : launch_any_h<T, BITS, false, kZeroAsym>(st, a);
  }
  if (!a.w_signed) return launch_any_h<T, BITS, false, kZeroSymU>(st, a);
  // (fp16 with 4-bit codes in an int8 container reaches this only off gemv_w4_m1's grid: rows
  // that are not whole multiples of 256 elements, groups shorter than 128)
  return launch_any_h<T, BITS, true, kZeroNone>(st, a);
}

}  // namespace

bool gemv_m1_any_supported(const LinearArgs& a) {
  if (a.m != 1 || (a.t_dtype != OFQ_F16 && a.t_dtype != OFQ_BF16)) return false;
  if ((a.bits != 4 && a.bits != 8) || a.group_dim != 1) return false;
  if (!a.symmetric && a.zero == nullptr) return false;
  const int epl = a.bits == 4 ? 32 : 16;  // elements behind a lane's 16 bytes of codes
  if (a.group_size < epl || log2_pow2(a.group_size) < 0 || a.k % a.group_size != 0) return false;
  // Rows of up to 4096 elements.  Beyond that the expansion of a row (3 to 6 vector instructions
  // per element, after the row has arrived) outweighs what the contiguous requests gain, and the
  // MFMA kernels, which leave the k-reduction to the matrix core, are faster (4096 x 11008, 4-bit
  // with a zero point: 7.7 us there against 10.4 us here).
  if (a.k % epl != 0 || a.k > 4096) return false;
  if (a.n < 1 || a.n > (1 << 24)) return false;
  if ((reinterpret_cast<uintptr_t>(a.x) & 15u) != 0 || (reinterpret_cast<uintptr_t>(a.w) & 15u) != 0) {
    return false;
  }
  return true;
}

int launch_gemv_m1_any(hipStream_t st, const LinearArgs& a) {
  if (!gemv_m1_any_supported(a)) return OFQ_ERR_UNSUPPORTED;
  if (a.t_dtype == OFQ_BF16) {
    return a.bits == 4 ? launch_any_scheme<bf16, 4>(st, a) : launch_any_scheme<bf16, 8>(st, a);
  }
  return a.bits == 4 ? launch_any_scheme<f16, 4>(st, a) : launch_any_scheme<f16, 8>(st, a);
}

}  // namespace ofq
