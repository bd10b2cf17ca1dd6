// MFMA GEMMs for gfx950:
//   (1) fused_linear_with_groupwise_quantized_weight for m > 16 ("prefill"): the weight tile is
//       dequantised on its way into LDS and feeds fp16/bf16 MFMA, so the fp16/bf16 copy of the
//       weight that the reference materialises for m > 8
//       (oneflow/core/functional/impl/quantization.cpp:341-350) never touches HBM;
//   (2) matmul_quant: int8 x int8 -> int32 MFMA with a per-row/per-tensor scale epilogue.
//
// Both are instances of one byte-oriented core.  A tile row is always 128 bytes of K
// (64 fp16/bf16 or 128 int8 elements), a k-step of the 32x32 MFMA consumes 32 of those bytes per
// row (16 bytes per lane), so the same LDS layout and fragment addressing serve every type.
//
//   block tile BM x BN, WM x WN waves, each wave owns (BM/WM) x (BN/WN) as 32x32 MFMA tiles;
//   LDS rows are padded from 128 to 144 bytes: the 16-byte fragment reads of 8 consecutive rows
//   then fall in 8 distinct 16-byte bank groups;
//   global -> register loads of tile kt+1 are issued before the MFMAs of tile kt, and LDS is
//   double buffered, so one barrier per k-tile suffices;
//   block ids are remapped so that the m-tiles sharing one weight tile run on the same XCD and
//   hit its L2.
#include "ofq_device.h"
#include "ofq_internal.h"

namespace ofq {
namespace {

constexpr int kRowBytes = 128;
constexpr int kLdsStride = 144;
constexpr int kThreads = 256;

// ---- MFMA policies -------------------------------------------------------------------------
struct MfmaF16 {
  typedef f32x16 Acc;
  static __device__ __forceinline__ Acc mma(u32x4 a, u32x4 b, Acc c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};
struct MfmaBF16 {
  typedef f32x16 Acc;
  static __device__ __forceinline__ Acc mma(u32x4 a, u32x4 b, Acc c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
struct MfmaI8 {
  typedef i32x16 Acc;
  static __device__ __forceinline__ Acc mma(u32x4 a, u32x4 b, Acc c) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, a),
                                                 __builtin_bit_cast(i32x4, b), c, 0, 0, 0);
  }
};

// ---- B-tile producers ------------------------------------------------------------------------
// Plain copy of 128-byte rows (int8 weights of matmul_quant).
template<int BN>
struct BCopy {
  struct Params {
    const uint8_t* b;
    int64_t ldb;  // bytes per row
    int N;
  };
  static constexpr int kChunks = BN * 8 / kThreads;
  struct Regs {
    u32x4 v[kChunks];
  };
  static __device__ __forceinline__ void load(const Params& p, int n0, int kt, int tid, Regs& r) {
#pragma unroll
    for (int i = 0; i < kChunks; ++i) {
      const int q = tid + i * kThreads;
      int row = n0 + (q >> 3);
      row = row < p.N ? row : p.N - 1;
      r.v[i] = *reinterpret_cast<const u32x4*>(p.b + (int64_t)row * p.ldb + (int64_t)kt * kRowBytes
                                               + (q & 7) * 16);
    }
  }
  static __device__ __forceinline__ void store(const Params&, const Regs& r, uint8_t* lds,
                                               int tid) {
#pragma unroll
    for (int i = 0; i < kChunks; ++i) {
      const int q = tid + i * kThreads;
      *reinterpret_cast<u32x4*>(lds + (q >> 3) * kLdsStride + (q & 7) * 16) = r.v[i];
    }
  }
};

// Groupwise-quantised weights: codes are loaded as they are stored ([N, K*bits/8] bytes), and
// turned into T with the reference arithmetic w~ = T(T(q)*s) + z when written to LDS.
template<typename T, int BITS, bool SIGNED, int ZMODE, int BN>
struct BDequant {
  struct Params {
    const uint8_t* w;
    const typename TT<T>::storage* scale;
    const typename TT<T>::storage* zero;
    int64_t ldw;  // bytes per row of codes
    int N;
    int G;           // groups per row
    int group_size;  // elements
  };
  static constexpr int kCodeBytesPerRow = 64 * BITS / 8;       // 64 elements of K per tile row
  static constexpr int kChunksPerRow = kCodeBytesPerRow / 16;  // 4 (8-bit) or 2 (4-bit)
  static constexpr int kElemsPerChunk = 16 * 8 / BITS;         // 16 or 32
  static constexpr int kChunks = BN * kChunksPerRow / kThreads;
  static_assert(kChunks >= 1, "tile too small for the thread count");
  struct Regs {
    u32x4 v[kChunks];
    float s[kChunks];
    float z[kChunks];
  };
  static __device__ __forceinline__ void load(const Params& p, int n0, int kt, int tid, Regs& r) {
#pragma unroll
    for (int i = 0; i < kChunks; ++i) {
      const int q = tid + i * kThreads;
      int row = n0 + q / kChunksPerRow;
      row = row < p.N ? row : p.N - 1;
      const int c = q % kChunksPerRow;
      r.v[i] = *reinterpret_cast<const u32x4*>(p.w + (int64_t)row * p.ldw
                                               + (int64_t)kt * kCodeBytesPerRow + c * 16);
      const int k = kt * 64 + c * kElemsPerChunk;
      const int64_t si = (int64_t)row * p.G + k / p.group_size;
      const float s = TT<T>::load(p.scale + si);
      r.s[i] = s;
      if (ZMODE == 2) {
        r.z[i] = TT<T>::load(p.zero + si);
      } else if (ZMODE == 1) {
        r.z[i] = TT<T>::round(-(float)((1 << (BITS - 1)) - 1) * s);
      } else {
        r.z[i] = 0.f;
      }
    }
  }
  static __device__ __forceinline__ void store(const Params&, const Regs& r, uint8_t* lds,
                                               int tid) {
    typedef typename TT<T>::storage S;
#pragma unroll
    for (int i = 0; i < kChunks; ++i) {
      const int q = tid + i * kThreads;
      const int row = q / kChunksPerRow;
      const int c = q % kChunksPerRow;
      S vals[kElemsPerChunk];
#pragma unroll
      for (int e = 0; e < kElemsPerChunk; ++e) {
        int code;
        if (BITS == 8) {
          const uint32_t b = (r.v[i][e >> 2] >> ((e & 3) * 8)) & 0xFFu;
          code = SIGNED ? (int)(int8_t)b : (int)b;
        } else {
          const uint32_t b = (r.v[i][e >> 3] >> (((e >> 1) & 3) * 8)) & 0xFFu;
          const int nib = (e & 1) ? (b & 0xF) : (b >> 4);
          code = SIGNED ? ((nib ^ 8) - 8) : nib;
        }
        float v = TT<T>::round((float)code * r.s[i]);
        if (ZMODE != 0) v = v + r.z[i];
        TT<T>::store(&vals[e], v);
      }
      uint8_t* dst = lds + row * kLdsStride + c * (kElemsPerChunk * 2);
#pragma unroll
      for (int j = 0; j < kElemsPerChunk * 2 / 16; ++j) {
        reinterpret_cast<u32x4*>(dst)[j] = reinterpret_cast<const u32x4*>(vals)[j];
      }
    }
  }
};

// ---- epilogues -------------------------------------------------------------------------------
template<typename T>
struct EpBias {
  struct Params {
    const typename TT<T>::storage* bias;
    typename TT<T>::storage* out;
  };
  static __device__ __forceinline__ void apply(const Params& p, float acc, int m, int n, int N) {
    if (p.bias != nullptr) acc += TT<T>::load(p.bias + n);
    TT<T>::store(p.out + (int64_t)m * N + n, acc);
  }
  static __device__ __forceinline__ float widen(float v) { return v; }
};
template<typename T>
struct EpScale {
  struct Params {
    const float* a_scale;
    const float* b_scale;
    const typename TT<T>::storage* bias;
    typename TT<T>::storage* out;
  };
  static __device__ __forceinline__ void apply(const Params& p, int acc, int m, int n, int N) {
    const float s = p.a_scale[0] * p.b_scale[n];
    float r = (float)acc * s;
    if (p.bias != nullptr) r = r + TT<T>::load(p.bias + n);
    TT<T>::store(p.out + (int64_t)m * N + n, r);
  }
};

// ---- the core ----------------------------------------------------------------------------------
template<class MF, class BP, class EP, int BM, int BN, int WM, int WN>
__global__ void __launch_bounds__(kThreads)
gemm_core(const uint8_t* __restrict__ A, int64_t lda, typename BP::Params bp,
          typename EP::Params ep, int M, int N, int KT, int m_tiles, int n_tiles) {
  static_assert(WM * WN * 64 == kThreads, "wave grid must match the block size");
  constexpr int WTM = BM / WM;  // wave tile
  constexpr int WTN = BN / WN;
  constexpr int TM = WTM / 32;
  constexpr int TN = WTN / 32;
  constexpr int kAChunks = BM * 8 / kThreads;
  constexpr int kABytes = BM * kLdsStride;
  constexpr int kBBytes = BN * kLdsStride;
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  // layout: [2][A tile | B tile]

  // XCD-aware tile order: hardware deals consecutive block ids round-robin to the 8 XCDs; give
  // each XCD a contiguous run of logical tiles, m fastest, so the m-tiles of one weight tile
  // share an L2.
  const int nblocks = m_tiles * n_tiles;
  int logical;
  {
    const int b = blockIdx.x;
    const int xcd = b & 7, idx = b >> 3;
    const int per = nblocks >> 3, rem = nblocks & 7;
    logical = xcd < rem ? xcd * (per + 1) + idx : rem * (per + 1) + (xcd - rem) * per + idx;
  }
  const int m0 = (logical % m_tiles) * BM;
  const int n0 = (logical / m_tiles) * BN;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm0 = (wave / WN) * WTM;
  const int wn0 = (wave % WN) * WTN;

  typename MF::Acc acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;

  u32x4 areg[kAChunks];
  typename BP::Regs breg;

  auto load_a = [&](int kt) {
#pragma unroll
    for (int i = 0; i < kAChunks; ++i) {
      const int q = tid + i * kThreads;
      int row = m0 + (q >> 3);
      row = row < M ? row : M - 1;
      areg[i] = *reinterpret_cast<const u32x4*>(A + (int64_t)row * lda + (int64_t)kt * kRowBytes
                                                + (q & 7) * 16);
    }
  };
  auto store_a = [&](uint8_t* dst) {
#pragma unroll
    for (int i = 0; i < kAChunks; ++i) {
      const int q = tid + i * kThreads;
      *reinterpret_cast<u32x4*>(dst + (q >> 3) * kLdsStride + (q & 7) * 16) = areg[i];
    }
  };

  load_a(0);
  BP::load(bp, n0, 0, tid, breg);

  const int frag_row = lane & 31;
  const int frag_col = (lane >> 5) * 16;

  for (int kt = 0; kt < KT; ++kt) {
    uint8_t* tile_a = lds + (kt & 1) * (kABytes + kBBytes);
    uint8_t* tile_b = tile_a + kABytes;
    store_a(tile_a);
    BP::store(bp, breg, tile_b, tid);
    __syncthreads();
    if (kt + 1 < KT) {
      load_a(kt + 1);
      BP::load(bp, n0, kt + 1, tid, breg);
    }
    const uint8_t* a_base = tile_a + (wm0 + frag_row) * kLdsStride + frag_col;
    const uint8_t* b_base = tile_b + (wn0 + frag_row) * kLdsStride + frag_col;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      u32x4 af[TM], bf[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        af[i] = *reinterpret_cast<const u32x4*>(a_base + i * 32 * kLdsStride + ks * 32);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        bf[j] = *reinterpret_cast<const u32x4*>(b_base + j * 32 * kLdsStride + ks * 32);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = MF::mma(af[i], bf[j], acc[i][j]);
    }
  }

  // D[row = 8*(v/4) + 4*(lane/32) + v%4][col = lane%32] of each 32x32 tile
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + wn0 + j * 32 + (lane & 31);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + wm0 + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        if (m < M && n < N) EP::apply(ep, acc[i][j][v], m, n, N);
      }
    }
  }
}

template<class MF, class BP, class EP, int BM, int BN, int WM, int WN>
int launch_core(hipStream_t st, const void* A, int64_t lda, const typename BP::Params& bp,
                const typename EP::Params& ep, int64_t M, int64_t N, int64_t KT) {
  const int m_tiles = (int)((M + BM - 1) / BM);
  const int n_tiles = (int)((N + BN - 1) / BN);
  const size_t lds_bytes = 2 * (size_t)(BM + BN) * kLdsStride;
  auto kern = gemm_core<MF, BP, EP, BM, BN, WM, WN>;
  if (lds_bytes > 48 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes)
        != hipSuccess) {
      return OFQ_ERR_LAUNCH;
    }
  }
  kern<<<m_tiles * n_tiles, kThreads, lds_bytes, st>>>(static_cast<const uint8_t*>(A), lda, bp, ep,
                                                       (int)M, (int)N, (int)KT, m_tiles, n_tiles);
  return ofq_check_launch();
}

template<typename T, class MF, int BITS, bool SIGNED, int ZMODE>
int launch_wq_variant(hipStream_t st, const LinearArgs& a) {
  typedef typename TT<T>::storage S;
  constexpr int BM = 128, BN = 128;
  typedef BDequant<T, BITS, SIGNED, ZMODE, BN> BP;
  typedef EpBias<T> EP;
  typename BP::Params bp;
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
  return launch_core<MF, BP, EP, BM, BN, 2, 2>(st, a.x, a.k * 2, bp, ep, a.m, a.n, a.k / 64);
}

template<typename T, class MF>
int launch_wq_t(hipStream_t st, const LinearArgs& a) {
  const int zmode = !a.symmetric ? 2 : (a.w_signed ? 0 : 1);
#define OFQ_V(B, SG, ZM)                                       \
  if (a.bits == B && a.w_signed == SG && zmode == ZM)          \
    return launch_wq_variant<T, MF, B, SG, ZM>(st, a);
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

int launch_gemm_wq(hipStream_t st, const LinearArgs& a) {
  if (a.t_dtype == OFQ_F16) return launch_wq_t<f16, MfmaF16>(st, a);
  return launch_wq_t<bf16, MfmaBF16>(st, a);
}

}  // namespace ofq

using namespace ofq;

extern "C" int ofq_matmul_quant(void* stream, const void* a, const void* b, const float* a_scale,
                                const float* b_scale, const void* bias, void* out, int out_dtype,
                                int64_t m, int64_t n, int64_t k) {
  OFQ_RETURN_IF(out_dtype != OFQ_F16 && out_dtype != OFQ_BF16 && out_dtype != OFQ_F32,
                OFQ_ERR_BAD_DTYPE);
  OFQ_RETURN_IF(m < 0 || n < 0 || k <= 0, OFQ_ERR_BAD_SHAPE);
  if (m == 0 || n == 0) return OFQ_OK;
  const int64_t i32max = 0x7FFFFFFF;
  OFQ_RETURN_IF(m * k > i32max || n * k > i32max || m * n > i32max, OFQ_ERR_UNSUPPORTED);
  // rows are consumed in 128-byte tiles of K
  OFQ_RETURN_IF(k % 128 != 0, OFQ_ERR_UNSUPPORTED);
  OFQ_RETURN_IF(a == nullptr || b == nullptr || a_scale == nullptr || b_scale == nullptr
                    || out == nullptr,
                OFQ_ERR_NULL_POINTER);
  OFQ_RETURN_IF(!ofq_aligned16(a) || !ofq_aligned16(b) || !ofq_aligned16(out), OFQ_ERR_MISALIGNED);
  hipStream_t st = static_cast<hipStream_t>(stream);
  constexpr int BM = 128, BN = 128;
  typedef BCopy<BN> BP;
  BP::Params bp;
  bp.b = static_cast<const uint8_t*>(b);
  bp.ldb = k;
  bp.N = (int)n;
#define OFQ_MQ(T)                                                                              \
  {                                                                                            \
    typedef EpScale<T> EP;                                                                     \
    EP::Params ep;                                                                             \
    ep.a_scale = a_scale;                                                                      \
    ep.b_scale = b_scale;                                                                      \
    ep.bias = static_cast<const TT<T>::storage*>(bias);                                        \
    ep.out = static_cast<TT<T>::storage*>(out);                                                \
    return launch_core<MfmaI8, BP, EP, BM, BN, 2, 2>(st, a, k, bp, ep, m, n, k / 128);         \
  }
  switch (out_dtype) {
    case OFQ_F16: OFQ_MQ(f16)
    case OFQ_BF16: OFQ_MQ(bf16)
    default: OFQ_MQ(float)
  }
#undef OFQ_MQ
}
