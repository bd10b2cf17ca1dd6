// Device code and launcher of the MFMA GEMM core shared by the prefill path of
// fused_linear_with_groupwise_quantized_weight and by matmul_quant.  Kept in a header so that
// experiments can instantiate tile configurations directly.
#pragma once

#include "ofq_device.h"

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

}  // namespace
}  // namespace ofq
