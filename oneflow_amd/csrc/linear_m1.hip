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

template<int NW, int H, int XU, int D = H>
int launch_m1_inst(hipStream_t st, const LinearArgs& a) {
  M1Shape sh;
  sh.N = (int)a.n;
  sh.K = (int)a.k;
  sh.rows_per_block = NW;  // one row per wave
  sh.gshift = log2_exact(a.group_size);
  sh.G = (int)(a.k / a.group_size);
  sh.gn = 1;
  const int grid = (int)((a.n + NW - 1) / NW);
  gemv_w4_m1<NW, 1, H, XU, D><<<grid, NW * 64, gemv_m1_lds_bytes(H), st>>>(
      static_cast<const f16*>(a.x), static_cast<const uint8_t*>(a.w),
      static_cast<const f16*>(a.scale), static_cast<const f16*>(a.bias), static_cast<f16*>(a.out),
      sh);
  return ofq_check_launch();
}

// many rows per wave: one block of 16 waves per CU, two from 128 rows per block on
template<int H>
int launch_m1_stream_inst(hipStream_t st, const LinearArgs& a) {
  constexpr int NW = 16;
  int grid = 256;
  if ((a.n + grid - 1) / grid >= 128) grid = 512;
  const int rpb = (int)((a.n + grid - 1) / grid);
  grid = (int)((a.n + rpb - 1) / rpb);
  M1Shape sh;
  sh.N = (int)a.n;
  sh.K = (int)a.k;
  sh.rows_per_block = rpb;
  sh.gshift = log2_exact(a.group_size);
  sh.G = (int)(a.k / a.group_size);
  sh.gn = 1;
  gemv_w4_m1_stream<NW, H, 1><<<grid, NW * 64, gemv_m1_lds_bytes(H), st>>>(
      static_cast<const f16*>(a.x), static_cast<const uint8_t*>(a.w),
      static_cast<const f16*>(a.scale), static_cast<const f16*>(a.bias), static_cast<f16*>(a.out),
      sh);
  return ofq_check_launch();
}

// groups along N: one row per wave, the block's rows inside one group
template<int NW, int H, int XU>
int launch_m1_gn_inst(hipStream_t st, const LinearArgs& a) {
  M1Shape sh;
  sh.N = (int)a.n;
  sh.K = (int)a.k;
  sh.rows_per_block = NW;
  sh.gshift = 0;
  sh.G = 0;
  sh.gn = (int)a.group_size;
  const int grid = (int)((a.n + NW - 1) / NW);
  gemv_w4_m1_gn<NW, H, XU><<<grid, NW * 64, gemv_m1_lds_bytes(H), st>>>(
      static_cast<const f16*>(a.x), static_cast<const uint8_t*>(a.w),
      static_cast<const f16*>(a.scale), static_cast<const f16*>(a.bias), static_cast<f16*>(a.out),
      sh);
  return ofq_check_launch();
}

template<int NW, int H, int XU>
int launch_m1_glu_inst(hipStream_t st, const LinearArgs& a, const M1Glu& glu) {
  M1Shape sh;
  sh.N = (int)a.n;
  sh.K = (int)a.k;
  sh.rows_per_block = NW;
  sh.gshift = log2_exact(a.group_size);
  sh.G = (int)(a.k / a.group_size);
  sh.gn = 1;
  const int grid = (int)((a.n + NW - 1) / NW);
  gemv_w4_m1_glu<NW, H, XU><<<grid, NW * 64, gemv_m1_lds_bytes(H), st>>>(
      static_cast<const f16*>(a.x), static_cast<const uint8_t*>(a.w),
      static_cast<const f16*>(a.scale), static_cast<const f16*>(a.bias), static_cast<f16*>(a.out),
      glu, sh);
  return ofq_check_launch();
}

template<int NW, int H, int XU>
int launch_m1_grouped_inst(hipStream_t st, const LinearArgs* pr, int count) {
  GemvGroup g{};
  g.count = count;
  int first = 0;
  for (int i = 0; i < count; ++i) {
    g.p[i].x = pr[i].x;
    g.p[i].w = static_cast<const uint8_t*>(pr[i].w);
    g.p[i].scale = pr[i].scale;
    g.p[i].zero = nullptr;
    g.p[i].bias = pr[i].bias;
    g.p[i].out = pr[i].out;
    g.p[i].N = (int)pr[i].n;
    g.p[i].first_block = first;
    first += (int)((pr[i].n + NW - 1) / NW);
  }
  M1Shape sh;
  sh.N = 0;  // per problem
  sh.K = (int)pr[0].k;
  sh.rows_per_block = NW;
  sh.gshift = log2_exact(pr[0].group_size);
  sh.G = (int)(pr[0].k / pr[0].group_size);
  sh.gn = 1;
  gemv_w4_m1_grouped<NW, H, XU><<<first, NW * 64, gemv_m1_lds_bytes(H), st>>>(g, sh);
  return ofq_check_launch();
}

// The fused GLU as a walk of (hidden, gate) row pairs: one block of 16 waves per CU.
template<int H>
int launch_m1_glu_walk_inst(hipStream_t st, const LinearArgs& a, const M1Glu& glu) {
  constexpr int NW = 16;
  const int rpb = (int)((a.n + 255) / 256);
  const int grid = (int)((a.n + rpb - 1) / rpb);
  M1Shape sh;
  sh.N = (int)a.n;
  sh.K = (int)a.k;
  sh.rows_per_block = rpb;
  sh.gshift = log2_exact(a.group_size);
  sh.G = (int)(a.k / a.group_size);
  sh.gn = 1;
  gemv_w4_m1_glu_walk<NW, H, 1><<<grid, NW * 64, gemv_m1_lds_bytes(H), st>>>(
      static_cast<const f16*>(a.x), static_cast<const uint8_t*>(a.w),
      static_cast<const f16*>(a.scale), static_cast<const f16*>(a.bias), static_cast<f16*>(a.out),
      glu, sh);
  return ofq_check_launch();
}

// Several problems as a walk: blocks of 12 waves, two per CU, every block inside one problem;
// rows per block = the smallest count that fits all problems into 512 blocks.
template<int H>
int launch_m1_grouped_walk_inst(hipStream_t st, const LinearArgs* pr, int count) {
  constexpr int NW = 12;
  int64_t total = 0;
  for (int i = 0; i < count; ++i) total += pr[i].n;
  int rpb = (int)((total + 511) / 512);
  auto blocks_at = [&](int r) {
    int64_t b = 0;
    for (int i = 0; i < count; ++i) b += (pr[i].n + r - 1) / r;
    return b;
  };
  while (blocks_at(rpb) > 512) ++rpb;
  GemvGroup g{};
  g.count = count;
  int first = 0;
  for (int i = 0; i < count; ++i) {
    g.p[i].x = pr[i].x;
    g.p[i].w = static_cast<const uint8_t*>(pr[i].w);
    g.p[i].scale = pr[i].scale;
    g.p[i].zero = nullptr;
    g.p[i].bias = pr[i].bias;
    g.p[i].out = pr[i].out;
    g.p[i].N = (int)pr[i].n;
    g.p[i].first_block = first;
    first += (int)((pr[i].n + rpb - 1) / rpb);
  }
  M1Shape sh;
  sh.N = 0;  // per problem
  sh.K = (int)pr[0].k;
  sh.rows_per_block = rpb;
  sh.gshift = log2_exact(pr[0].group_size);
  sh.G = (int)(pr[0].k / pr[0].group_size);
  sh.gn = 1;
  gemv_w4_m1_grouped_walk<NW, H, 1><<<first, NW * 64, gemv_m1_lds_bytes(H), st>>>(g, sh);
  return ofq_check_launch();
}

// picks the instance for k: NW = 16 up to 2 KB of codes per row, 8 beyond
#define OFQ_M1_DISPATCH(k, CALL)                      \
  do {                                                \
    const int h_ = (int)(((k) / 2 + 1023) / 1024);    \
    if ((k) <= 4096) {                                \
      if (h_ == 1) return CALL(16, 1, 1);             \
      return CALL(16, 2, 1);                          \
    }                                                 \
    switch (h_) {                                     \
      case 3: return CALL(8, 3, 1);                   \
      case 4: return CALL(8, 4, 1);                   \
      case 5: return CALL(8, 5, 2);                   \
      case 6: return CALL(8, 6, 2);                   \
      case 7: return CALL(8, 7, 2);                   \
      case 8: return CALL(8, 8, 2);                   \
      default: return OFQ_ERR_UNSUPPORTED;            \
    }                                                 \
  } while (0)

}  // namespace

bool gemv_m1_supported(const LinearArgs& a) {
  return a.m == 1 && a.t_dtype == OFQ_F16 && a.bits == 4 && a.w_signed && a.symmetric
         && a.group_dim == 1 && a.group_size >= 128 && log2_exact(a.group_size) >= 0
         && a.k % 256 == 0 && a.k <= 16384 && a.k % a.group_size == 0 && a.n >= 1
         && a.n <= (1 << 24);
}

// Blocks of 16 waves when a row is at most 2 KB of codes (k <= 4096): with short rows a second
// staging of x costs more than two small blocks gain (4096 x 4096: 3.55 against 3.8 us).  Longer
// rows: 16 waves with 3 KB of the row requested ahead when the blocks fill the chip (n >= 3072),
// otherwise blocks of 8 waves with the whole row requested up front (2048 x 11008: 4.5 against
// 4.85 us; with everything requested up front two small blocks per CU, each with its own
// barrier, run ahead of one large one, 4096 x 11008: 6.3 against 6.7 us).
// One row per wave while one resident round of blocks covers n (n <= 4096); beyond that, for rows
// of at most 2 KB of codes, the streaming kernel (11008 x 4096: 6.2 against 6.4 us; 128256 x
// 4096: 41.5 against 50 us, 6.5 TB/s).
int launch_gemv_m1(hipStream_t st, const LinearArgs& a) {
  if (a.n > 4096 && a.k <= 4096) {
    return a.k <= 2048 ? launch_m1_stream_inst<1>(st, a) : launch_m1_stream_inst<2>(st, a);
  }
  if (a.k > 4096 && a.n >= 3072) {
    switch ((int)((a.k / 2 + 1023) / 1024)) {
      case 3: return launch_m1_inst<16, 3, 1, 2>(st, a);
      case 4: return launch_m1_inst<16, 4, 1, 3>(st, a);
      case 5: return launch_m1_inst<16, 5, 1, 3>(st, a);
      case 6: return launch_m1_inst<16, 6, 1, 3>(st, a);
      case 7: return launch_m1_inst<16, 7, 1, 3>(st, a);
      case 8: return launch_m1_inst<16, 8, 1, 3>(st, a);
      default: return OFQ_ERR_UNSUPPORTED;
    }
  }
#define OFQ_M1_PLAIN(NW, H, XU) launch_m1_inst<NW, H, XU>(st, a)
  OFQ_M1_DISPATCH(a.k, OFQ_M1_PLAIN);
#undef OFQ_M1_PLAIN
}

// Groups along N (scale [n / group_size, k]): the scale is applied to x once per block.
bool gemv_m1_gn_supported(const LinearArgs& a) {
  return a.m == 1 && a.t_dtype == OFQ_F16 && a.bits == 4 && a.w_signed && a.symmetric
         && a.group_dim == 0 && a.group_size % 16 == 0 && a.n % a.group_size == 0
         && a.k % 256 == 0 && a.k <= 16384 && a.n >= 1 && a.n <= (1 << 24)
         && (reinterpret_cast<uintptr_t>(a.scale) & 15u) == 0
         && (reinterpret_cast<uintptr_t>(a.x) & 15u) == 0
         && (reinterpret_cast<uintptr_t>(a.w) & 15u) == 0;
}

int launch_gemv_m1_gn(hipStream_t st, const LinearArgs& a) {
  if (!gemv_m1_gn_supported(a)) return OFQ_ERR_UNSUPPORTED;
#define OFQ_M1_GN(NW, H, XU) launch_m1_gn_inst<NW, H, XU>(st, a)
  OFQ_M1_DISPATCH(a.k, OFQ_M1_GN);
#undef OFQ_M1_GN
}

// Two weights of equal shape on one x (hidden, gate) + the gating, one launch.
int launch_gemv_m1_glu(hipStream_t st, const LinearArgs& a, const LinearArgs& g, void* y, int act) {
  if (!gemv_m1_supported(a) || !gemv_m1_supported(g)) return OFQ_ERR_UNSUPPORTED;
  if (g.n != a.n || g.k != a.k || g.x != a.x || g.group_size != a.group_size) {
    return OFQ_ERR_UNSUPPORTED;
  }
  M1Glu glu;
  glu.w2 = static_cast<const uint8_t*>(g.w);
  glu.scale2 = static_cast<const f16*>(g.scale);
  glu.bias2 = static_cast<const f16*>(g.bias);
  glu.out2 = static_cast<f16*>(g.out);
  glu.y = static_cast<f16*>(y);
  glu.act = act;
  // beyond one resident round of one-pair-per-wave blocks (8192 rows of the two weights): the walk
  if (a.k <= 4096 && a.n > 4096) {
    return a.k <= 2048 ? launch_m1_glu_walk_inst<1>(st, a, glu)
                       : launch_m1_glu_walk_inst<2>(st, a, glu);
  }
#define OFQ_M1_GLU(NW, H, XU) launch_m1_glu_inst<NW, H, XU>(st, a, glu)
  OFQ_M1_DISPATCH(a.k, OFQ_M1_GLU);
#undef OFQ_M1_GLU
}

// Up to kGemvMaxProblems problems of equal k and group size, one launch.
int launch_gemv_m1_grouped(hipStream_t st, const LinearArgs* pr, int count) {
  if (count < 1 || count > kGemvMaxProblems) return OFQ_ERR_UNSUPPORTED;
  int64_t blocks = 0;
  for (int i = 0; i < count; ++i) {
    if (!gemv_m1_supported(pr[i]) || pr[i].k != pr[0].k || pr[i].group_size != pr[0].group_size) {
      return OFQ_ERR_UNSUPPORTED;
    }
    blocks += (pr[i].n + 7) / 8;
  }
  if (blocks > 0x7FFFFFFF) return OFQ_ERR_UNSUPPORTED;
  {
    int64_t total = 0;
    for (int i = 0; i < count; ++i) total += pr[i].n;
    // more rows than one resident round of one-row-per-wave blocks (2 x 256 x 16) holds
    if (pr[0].k <= 4096 && total > 8192) {
      return pr[0].k <= 2048 ? launch_m1_grouped_walk_inst<1>(st, pr, count)
                             : launch_m1_grouped_walk_inst<2>(st, pr, count);
    }
  }
#define OFQ_M1_GROUPED(NW, H, XU) launch_m1_grouped_inst<NW, H, XU>(st, pr, count)
  OFQ_M1_DISPATCH(pr[0].k, OFQ_M1_GROUPED);
#undef OFQ_M1_GROUPED
}

}  // namespace ofq
