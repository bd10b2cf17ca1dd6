// Device code and launcher of the MFMA GEMM core shared by the prefill path of
// fused_linear_with_groupwise_quantized_weight and by matmul_quant.  Kept in a header so that
// experiments can instantiate tile configurations directly.
#pragma once

#include <atomic>
#include <type_traits>
#include "dequant_regs.h"
#include "ofq_device.h"

namespace ofq {
namespace {

// ---- MFMA policies -------------------------------------------------------------------------
struct MfmaF16 {
  typedef f32x16 Acc;
  typedef float Scalar;
  static __device__ __forceinline__ Acc mma(u32x4 a, u32x4 b, Acc c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};
struct MfmaBF16 {
  typedef f32x16 Acc;
  typedef float Scalar;
  static __device__ __forceinline__ Acc mma(u32x4 a, u32x4 b, Acc c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
struct MfmaI8 {
  typedef i32x16 Acc;
  typedef int Scalar;
  static __device__ __forceinline__ Acc mma(u32x4 a, u32x4 b, Acc c) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, a),
                                                 __builtin_bit_cast(i32x4, b), c, 0, 0, 0);
  }
};

// ---- B-tile producers ------------------------------------------------------------------------
// Plain copy of 128-byte rows (int8 weights of matmul_quant).
struct BCopyParams {
  const uint8_t* b;
  int64_t ldb;  // bytes per row
  int N;
};
// Groupwise-quantised weights [N, K*bits/8] with scale / zero [N, G] in T
template<typename T>
struct WqParams {
  const uint8_t* w;
  const typename TT<T>::storage* scale;
  const typename TT<T>::storage* zero;
  int64_t ldw;  // bytes per row of codes
  int N;
  int G;           // groups per row
  int group_size;  // elements
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
  // four consecutive n (n .. n+3, all < N): bias added in fp32, one rounding to T
  static __device__ __forceinline__ void convert4(const Params& p, const float* acc, int n,
                                                  typename TT<T>::storage* out4) {
    typename TT<T>::storage bias4[4];
    if (p.bias != nullptr) {
      if (sizeof(typename TT<T>::storage) == 2) {
        *reinterpret_cast<u32x2*>(bias4) = *reinterpret_cast<const u32x2*>(p.bias + n);
      } else {
        *reinterpret_cast<u32x4*>(bias4) = *reinterpret_cast<const u32x4*>(p.bias + n);
      }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float v = acc[e];
      if (p.bias != nullptr) v += TT<T>::load(bias4 + e);
      TT<T>::store(out4 + e, v);
    }
  }
  static __device__ __forceinline__ typename TT<T>::storage convert1(const Params& p, float acc,
                                                                     int n) {
    typename TT<T>::storage o;
    if (p.bias != nullptr) acc += TT<T>::load(p.bias + n);
    TT<T>::store(&o, acc);
    return o;
  }
  typedef T elem_t;
  static constexpr bool kSplit = false;
};
// Split-K: the block's fp32 partial sums go to slice blockIdx.y of a [splits, M, N] workspace;
// a second kernel adds the slices in order and applies the real epilogue.
struct EpPartial {
  struct Params {
    float* out;
  };
  static __device__ __forceinline__ void convert4(const Params&, const float* acc, int,
                                                  float* out4) {
#pragma unroll
    for (int e = 0; e < 4; ++e) out4[e] = acc[e];
  }
  static __device__ __forceinline__ float convert1(const Params&, float acc, int) { return acc; }
  typedef float elem_t;
  static constexpr bool kSplit = true;
};
// Split-K of the int8 GEMM: the int32 partial sums go to the workspace bit for bit (the slot type
// is float only because the epilogue's stores are typed by 4-byte elements; nothing is converted).
struct EpPartialI32 {
  struct Params {
    float* out;
  };
  static __device__ __forceinline__ void convert4(const Params&, const int* acc, int,
                                                  float* out4) {
#pragma unroll
    for (int e = 0; e < 4; ++e) out4[e] = __builtin_bit_cast(float, acc[e]);
  }
  static __device__ __forceinline__ float convert1(const Params&, int acc, int) {
    return __builtin_bit_cast(float, acc);
  }
  typedef float elem_t;
  static constexpr bool kSplit = true;
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
  // n is a multiple of 4: the four scales (and biases) come as one aligned vector load
  static __device__ __forceinline__ void convert4(const Params& p, const int* acc, int n,
                                                  typename TT<T>::storage* out4) {
    const float sa = p.a_scale[0];
    const f32x4 sb = *reinterpret_cast<const f32x4*>(p.b_scale + n);
    typename TT<T>::storage bias4[4];
    if (p.bias != nullptr) {
      if (sizeof(typename TT<T>::storage) == 2) {
        *reinterpret_cast<u32x2*>(bias4) = *reinterpret_cast<const u32x2*>(p.bias + n);
      } else {
        *reinterpret_cast<u32x4*>(bias4) = *reinterpret_cast<const u32x4*>(p.bias + n);
      }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float s = sa * sb[e];
      float r = (float)acc[e] * s;
      if (p.bias != nullptr) r = r + TT<T>::load(bias4 + e);
      TT<T>::store(out4 + e, r);
    }
  }
  static __device__ __forceinline__ typename TT<T>::storage convert1(const Params& p, int acc,
                                                                     int n) {
    typename TT<T>::storage o;
    float r = (float)acc * (p.a_scale[0] * p.b_scale[n]);
    if (p.bias != nullptr) r = r + TT<T>::load(p.bias + n);
    TT<T>::store(&o, r);
    return o;
  }
  typedef T elem_t;
  static constexpr bool kSplit = false;
};

// =================================================================================================
// The core: asynchronous global->LDS copies (global_load_lds_dwordx4) for every tile
// that needs no arithmetic on the way, XOR-swizzled 128-byte LDS rows instead of padding, two LDS
// stages with the copies issued one full k-tile ahead, and (for quantised weights) the codes
// fetched two k-tiles ahead into registers and dequantised into LDS in the shadow of the MFMAs.
//
// What bounds it: the path L2 -> vector L1 -> LDS delivers 64 bytes per clock per CU, and a k-tile
// of a BM x BN block needs (BM+BN)*128 bytes for BM*BN/32 MFMA clocks per SIMD.  128x128 needs
// exactly 64 B/clk at full MFMA rate, 256x128 needs 48, 256x256 needs 32 -- large tiles are not a
// register-reuse nicety here but the condition for being MFMA-bound at all.
//
// LDS addressing.  A wave-level global_load_lds writes 64 x 16 bytes to consecutive LDS addresses,
// i.e. 8 rows of 128 bytes.  Lane l fills slot (row = l/8, position p = l%8) and fetches the
// global 16-byte piece c = p ^ key(row) of its row, key(r) = (r >> 1) & 7, so piece c of row r
// lives at position c ^ key(r).  gfx950's LDS serves 256 bytes per clock: a ds_read_b128 retires
// 16 lanes at a time and those must fall into 16 different 16-byte bank groups (address bits
// 4..7 = position + 8 * (row & 1)).  The fragment reads of 16 consecutive rows (same c) see
// every key twice, once per row parity: conflict-free without padding.  (Keying on row & 7
// instead costs a two-way conflict on every fragment read: measured, half the LDS cycles.)
// =================================================================================================
constexpr int kStageRow = 128;
__device__ __forceinline__ int swizzle_key(int row) { return (row >> 1) & 7; }

// One wave-level global -> LDS copy (global_load_lds_dwordx4): 64 lanes x 16 bytes to consecutive
// LDS addresses from lds_addr_uniform on.  The address is split by hand, scalar base + 32-bit lane
// offset, LDS address in M0, and the instruction is written as assembly, for two measured
// reasons.  (1) Through the builtin the split is left to the loop optimiser, which turns the
// loop-invariant lane offsets into 64-bit pointers carried from k-tile to k-tile: two registers per
// request in a kernel that has none to spare.  (2) While a copy issued through the builtin is in
// flight the compiler's wait insertion treats every later LDS read as unordered and waits with
// lgkmcnt(0), i.e. for the request it has just issued; not knowing about the copy, it counts the
// fragment reads exactly (lgkmcnt(6), (5), ...) and the reads of one k-step overlap the matrix
// instructions of the step before.  2048 x 11008 x 4096: bf16 176 -> 157 us, int8 117 -> 108 us on
// random operands.  The kernel waits for its copies by hand (wait_vmem_le / wait_vmem_all below) and
// a barrier, as it did before.  Every copy of a kernel must come through here: the compiler is
// told that M0 changes, not what it holds.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"  // "clobber list contains reserved registers: m0"
__device__ __forceinline__ void async_copy16_at(const uint8_t* base_uniform, uint32_t lane_off,
                                                uint32_t lds_addr_uniform) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(lane_off), "s"(base_uniform), "s"(lds_addr_uniform)
               : "memory", "m0");
}
#pragma clang diagnostic pop
// wait until at most N of this wave's vector-memory operations (incl. global->LDS copies) are
// still outstanding; they complete in issue order, so this retires everything but the N newest
template<int N>
__device__ __forceinline__ void wait_vmem_le() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 0xF) | ((N >> 4) << 14));
}
__device__ __forceinline__ void wait_vmem_all() { wait_vmem_le<0>(); }

// rows [0, ROWS) x 128 bytes of tile kt of a row-major byte matrix -> swizzled LDS tile
template<int ROWS, int NWAVES>
__device__ __forceinline__ void async_tile(const uint8_t* __restrict__ g, int64_t ld, int row0,
                                           int row_limit, int kt, uint8_t* lds_tile, int wave,
                                           int lane) {
  static_assert(ROWS % 8 == 0, "tile rows come in groups of 8");
  constexpr int kGroups = ROWS / 8;
  const int sub = lane >> 3;  // row within the 8-row group
  // wave-uniform part of the address (scalar registers) + a 32-bit offset per lane that does not
  // change from k-tile to k-tile: one vector register per request instead of a 64-bit pointer
  // (the tile's rows span less than 4 GB: checked by the launcher)
  const uint8_t* gk = g + (int64_t)row0 * ld + (int64_t)kt * kStageRow;
  const uint32_t lds0 =
      (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds_tile;
#pragma unroll
  for (int j = 0; j < (kGroups + NWAVES - 1) / NWAVES; ++j) {
    const int grp = j * NWAVES + wave;  // 8-row group of the tile (wave-uniform)
    if (kGroups % NWAVES != 0 && grp >= kGroups) break;
    const int piece = (lane & 7) ^ swizzle_key(grp * 8 + sub);  // global piece this lane fetches
    int rel = grp * 8 + sub;  // row within the tile; rows past the matrix repeat its last row
    rel = row0 + rel < row_limit ? rel : row_limit - 1 - row0;
    const uint32_t off = (uint32_t)rel * (uint32_t)ld + (uint32_t)(piece * 16);
    async_copy16_at(gk, off, lds0 + grp * 1024);
  }
}

template<int BN, int NT>
struct B2Copy {
  typedef BCopyParams Params;
  static constexpr bool kDirect = true;
  struct Regs {};
  static __device__ __forceinline__ void load(const Params& p, int n0, int kt, int wave, int lane,
                                              int, Regs&, uint8_t* lds_b) {
    async_tile<BN, NT / 64>(p.b, p.ldb, n0, p.N, kt, lds_b, wave, lane);
  }
  static __device__ __forceinline__ void store_part(const Params&, const Regs&, uint8_t*, int, int) {}
};

// Groupwise-quantised weights: codes are loaded as stored
// ([N, K*bits/8] bytes) two k-tiles ahead, and turned into T when written to the swizzled LDS tile.
template<typename T, int BITS, bool SIGNED, int ZMODE, int BN, int NT>
struct B2Dequant {
  typedef WqParams<T> Params;
  static constexpr bool kDirect = false;
  static constexpr int kCodeBytesPerRow = 64 * BITS / 8;
  static constexpr int kChunksPerRow = kCodeBytesPerRow / 16;  // 4 (8-bit) or 2 (4-bit)
  static constexpr int kElemsPerChunk = 16 * 8 / BITS;         // 16 or 32
  static constexpr int kTotalChunks = BN * kChunksPerRow;
  static constexpr int kChunks = (kTotalChunks + NT - 1) / NT;
  static constexpr bool kRagged = kTotalChunks % NT != 0;  // some threads own one chunk less
  // scale / zero stay in their storage type until they are used: converting them at load time
  // would put a wait for the loads right behind their issue
  struct Regs {
    u32x4 v[kChunks];
    // raw 16 bits each.  With a zero term or 8-bit codes they get registers of their own:
    // 16-bit slots there ended up in scratch memory (a store and two loads per k-tile).
    typedef typename std::conditional<BITS == 4 && ZMODE == 0, uint16_t, uint32_t>::type Slot;
    Slot s[kChunks];
    Slot z[kChunks];
  };
  static __device__ __forceinline__ void load(const Params& p, int n0, int kt, int, int, int tid,
                                              Regs& r, uint8_t*) {
#pragma unroll
    for (int i = 0; i < kChunks; ++i) {
      const int q = tid + i * NT;
      if (kRagged && q >= kTotalChunks) continue;
      int row = n0 + q / kChunksPerRow;
      row = row < p.N ? row : p.N - 1;
      const int c = q % kChunksPerRow;
      r.v[i] = *reinterpret_cast<const u32x4*>(p.w + (int64_t)row * p.ldw
                                               + (int64_t)kt * kCodeBytesPerRow + c * 16);
      const int k = kt * 64 + c * kElemsPerChunk;
      const int64_t si = (int64_t)row * p.G + k / p.group_size;
      r.s[i] = reinterpret_cast<const uint16_t*>(p.scale)[si];
      if (ZMODE == 2) r.z[i] = reinterpret_cast<const uint16_t*>(p.zero)[si];
    }
  }
  // dequantise and store a quarter of the thread's chunks (all of them when there are fewer)
  static __device__ __forceinline__ void store_part(const Params&, const Regs& r, uint8_t* lds,
                                                    int tid, int part) {
#pragma unroll
    for (int i = 0; i < kChunks; ++i) {
      if ((kChunks >= 4 ? (i & 3) : (i * (4 / kChunks))) != part) continue;
      const int q = tid + i * NT;
      if (kRagged && q >= kTotalChunks) continue;
      const int row = q / kChunksPerRow;
      const int c = q % kChunksPerRow;
      uint8_t* rowp = lds + row * kStageRow;
      const int sw = swizzle_key(row);
      const float sc = raw16_to_float<T>((uint16_t)r.s[i]);
      float zc = 0.f;
      if (ZMODE == 2) zc = raw16_to_float<T>((uint16_t)r.z[i]);
      if (ZMODE == 1) zc = TT<T>::round(-(float)((1 << (BITS - 1)) - 1) * sc);
      if constexpr (BITS == 8) {
        u32x4 o0, o1;
        dequant16_b8<T, SIGNED, ZMODE>(r.v[i], sc, zc, o0, o1);
        *reinterpret_cast<u32x4*>(rowp + (((2 * c) ^ sw) << 4)) = o0;
        *reinterpret_cast<u32x4*>(rowp + (((2 * c + 1) ^ sw) << 4)) = o1;
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          *reinterpret_cast<u32x4*>(rowp + (((4 * c + j) ^ sw) << 4)) =
              dequant8_b4<T, SIGNED, ZMODE>(r.v[i][j], sc, zc);
      }
    }
  }
};

// NSTAGE LDS stages; the copies of tile t are issued at the top of iteration t-(NSTAGE-1).
template<class MF, class BP, class EP, int BM, int BN, int WM, int WN, int NSTAGE = 2>
__global__ void __launch_bounds__(WM * WN * 64)
gemm_core2(const uint8_t* __restrict__ A, int64_t lda, typename BP::Params bp,
           typename EP::Params ep, int M, int N, int KT_total, int kt_split, int m_tiles,
           int n_tiles) {
  constexpr int NWAVES = WM * WN;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int kABytes = BM * kStageRow;
  constexpr int kStage = (BM + BN) * kStageRow;
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

  // split-K: blockIdx.y owns k-tiles [kt_base, kt_base + KT); tile t below is the block's t-th
  const int kt_base = EP::kSplit ? (int)blockIdx.y * kt_split : 0;
  const int KT = EP::kSplit ? (KT_total - kt_base < kt_split ? KT_total - kt_base : kt_split)
                            : KT_total;
  if (EP::kSplit) ep.out += (int64_t)blockIdx.y * M * N;

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
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave / WN) * WTM;
  const int wn0 = (wave % WN) * WTN;

  typename MF::Acc acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;

  typename BP::Regs breg0, breg1;  // codes of even / odd tiles (never indexed dynamically)
  constexpr int D = NSTAGE - 1;  // prefetch distance of the copies
  // vector-memory operations a wave issues per iteration for the copies (they are issued last,
  // so "at most this many outstanding" means: everything older has landed)
  static_assert(NSTAGE == 2 || (BM % (8 * NWAVES) == 0 && BN % (8 * NWAVES) == 0),
                "deeper pipelines need the same number of copies in every wave");
  constexpr int kCopyOps = BM / (8 * NWAVES) + (BP::kDirect ? BN / (8 * NWAVES) : 0);
  auto stage_of = [&](int t) { return lds + (t % NSTAGE) * kStage; };
  auto issue_copies = [&](int t, typename BP::Regs& regs) {
    async_tile<BM, NWAVES>(A, lda, m0, M, kt_base + t, stage_of(t), wave, lane);
    if (BP::kDirect) BP::load(bp, n0, kt_base + t, wave, lane, tid, regs, stage_of(t) + kABytes);
  };

  // ---- prologue: tile 0 complete in its stage, copies of tiles 1..D-1 and the codes of tile 1
  //      in flight --------------------------------------------------------------------------------
  if (!BP::kDirect) {
    BP::load(bp, n0, kt_base, wave, lane, tid, breg0, nullptr);
#pragma unroll
    for (int part = 0; part < 4; ++part) BP::store_part(bp, breg0, lds + kABytes, tid, part);
    if (KT > 1) BP::load(bp, n0, kt_base + 1, wave, lane, tid, breg1, nullptr);
  }
  issue_copies(0, breg0);
  wait_vmem_all();
#pragma unroll
  for (int t = 1; t < D; ++t)
    if (t < KT) issue_copies(t, breg0);
  __syncthreads();

  // fragment addressing: row = (wave tile row) + i*32 + lane%32, piece c = 2*ks + lane/32 stored
  // at position c ^ key(row); key(row) depends on the lane only because every tile origin is a
  // multiple of 16
  const int frag_row = lane & 31;
  const int x7 = swizzle_key(frag_row);
  const int half = lane >> 5;
  int frag_off[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) frag_off[ks] = ((2 * ks + half) ^ x7) << 4;

  // One k-tile.  On entry every wave has passed the barrier that ended iteration kt-1, tile kt is
  // complete in its stage and the stage of tile kt-1 is free.  `st_regs` holds the codes of tile
  // kt+1 (requested at the top of iteration kt-1); they are dequantised into that tile's stage
  // during the MFMAs.  `ld_regs` (free since iteration kt-1) receives the codes of tile kt+2.
  // Issue order per iteration: code loads first, copies last, so that "at most kCopyOps
  // outstanding" at the end retires everything except the copies just issued.
  auto iteration = [&](int kt, typename BP::Regs& st_regs, typename BP::Regs& ld_regs) {
    const bool more_copies = kt + D < KT;
    if (!BP::kDirect && kt + 2 < KT)
      BP::load(bp, n0, kt_base + kt + 2, wave, lane, tid, ld_regs, nullptr);
    if (more_copies) issue_copies(kt + D, ld_regs);
    uint8_t* cur = stage_of(kt);
    uint8_t* nxt = stage_of(kt + 1);
    const uint8_t* a_base = cur + (wm0 + frag_row) * kStageRow;
    const uint8_t* b_base = cur + kABytes + (wn0 + frag_row) * kStageRow;
    const bool store_b = !BP::kDirect && (kt + 1 < KT);
    // fragments of k-step ks+1 are fetched before the MFMAs of k-step ks are issued (when the
    // fragment set is small enough to keep twice in registers)
    constexpr bool kDoubleFrag = (TM + TN) <= 6;
    u32x4 af[2][TM], bf[2][TN];
    auto fetch = [&](int ks, int set) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
        af[set][i] = *reinterpret_cast<const u32x4*>(a_base + i * 32 * kStageRow + frag_off[ks]);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        bf[set][j] = *reinterpret_cast<const u32x4*>(b_base + j * 32 * kStageRow + frag_off[ks]);
    };
    if (kDoubleFrag) fetch(0, 0);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const int set = kDoubleFrag ? (ks & 1) : 0;
      if (kDoubleFrag) {
        if (ks < 3) fetch(ks + 1, (ks + 1) & 1);
      } else {
        fetch(ks, 0);
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          // weights as the first operand: the 32x32 result is D[n][m], so a lane ends up with
          // 4 CONSECUTIVE n per register quad -- what the row-major output wants
          acc[i][j] = MF::mma(bf[set][j], af[set][i], acc[i][j]);
        }
      // a quarter of the conversions per k-step, in the shadow of the MFMAs just issued
      if (store_b) BP::store_part(bp, st_regs, nxt + kABytes, tid, ks);
    }
    // tile kt+1 must be complete: its copies are older than those issued in this iteration
    if (D > 1 && more_copies) {
      wait_vmem_le<kCopyOps>();
    } else {
      wait_vmem_all();
    }
    __syncthreads();  // ... for every wave, and everyone is done reading `cur`
  };
  for (int kt = 0; kt < KT; kt += 2) {
    iteration(kt, breg1, breg0);
    if (kt + 1 < KT) iteration(kt + 1, breg0, breg1);
  }

  // ---- epilogue: registers -> (wave-private, padded) LDS tile -> 128-bit row-contiguous stores --
  // Each lane holds, per 32x32 tile and register quad g, the 4 consecutive outputs
  // out[m = .. + lane%32][n = .. + 8g + 4*(lane/32) + 0..3]; they are converted (bias / scales,
  // one rounding to T), packed to 8 bytes and written to LDS; rows are then read back 16 bytes
  // per lane so that every global store instruction writes whole row segments.
  typedef typename EP::elem_t OT;
  typedef typename TT<OT>::storage OS;
  static_assert(sizeof(OS) == 2 || sizeof(OS) == 4, "output element size");
  // The wave tile is written in panels of JP 32-column MFMA tiles so that the staging area of all
  // waves fits in the stage memory.
  constexpr int kLdsBudget = NSTAGE * kStage;
  constexpr int JP0 = (kLdsBudget / (NWAVES * WTM) - 8) / (32 * (int)sizeof(OS));
  constexpr int JP = JP0 >= TN ? TN : (JP0 >= 4 ? (JP0 / 2) * 2 : JP0);  // whole 128-byte pieces
  static_assert(JP >= 1, "no room for the epilogue staging area");
  constexpr int kRowBytesOut = JP * 32 * (int)sizeof(OS) + 8;  // +8: conflict-free 8-byte writes
  uint8_t* ep_tile = lds + wave * (WTM * kRowBytesOut);  // all waves passed the last barrier
#pragma unroll
  for (int jp = 0; jp < TN; jp += JP) {
    const int panel_cols = (TN - jp < JP ? TN - jp : JP) * 32;
    const int ncol0 = n0 + wn0 + jp * 32;  // first column of the panel
    const bool vec_ok = (N % 8 == 0) && (ncol0 + panel_cols <= N);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int jj = 0; jj < JP; ++jj) {
        const int j = jp + jj;
        if (j >= TN) break;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int nl = jj * 32 + 8 * g + 4 * (lane >> 5);  // column of the quad in the panel
          const int n = ncol0 + nl;
          OS q[4];
          typename MF::Acc& a = acc[i][j];
          if (n + 3 < N) {
            const typename MF::Scalar quad[4] = {a[4 * g], a[4 * g + 1], a[4 * g + 2], a[4 * g + 3]};
            EP::convert4(ep, quad, n, q);
          } else {
            // quad straddles or lies beyond N: element-wise, out-of-range slots are never stored
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              q[e] = OS();
              if (n + e < N) q[e] = EP::convert1(ep, a[4 * g + e], n + e);
            }
          }
          uint8_t* dst = ep_tile + (i * 32 + (lane & 31)) * kRowBytesOut + nl * (int)sizeof(OS);
          if (sizeof(OS) == 2) {
            *reinterpret_cast<u32x2*>(dst) = *reinterpret_cast<const u32x2*>(q);
          } else {
            *reinterpret_cast<u32x2*>(dst) = reinterpret_cast<const u32x2*>(q)[0];
            *reinterpret_cast<u32x2*>(dst + 8) = reinterpret_cast<const u32x2*>(q)[1];
          }
        }
      }
    }
    // a wave only reads what it wrote itself; LDS operations of one wave complete in order.
    // 16 bytes per lane: piece p of row r, pieces_per_row = panel bytes / 16.
    const int pieces_per_row = panel_cols * (int)sizeof(OS) / 16;
    const int total_pieces = WTM * pieces_per_row;
    for (int t = lane; t < total_pieces; t += 64) {
      const int ml = t / pieces_per_row;
      const int cpiece = t - ml * pieces_per_row;
      const int m = m0 + wm0 + ml;
      if (m >= M) continue;
      const uint8_t* src = ep_tile + ml * kRowBytesOut + cpiece * 16;
      const u32x2 lo = *reinterpret_cast<const u32x2*>(src);
      const u32x2 hi = *reinterpret_cast<const u32x2*>(src + 8);
      const int ncol = ncol0 + cpiece * (16 / (int)sizeof(OS));
      OS* gdst = ep.out + (int64_t)m * N + ncol;
      const u32x4 v = {lo[0], lo[1], hi[0], hi[1]};
      if (vec_ok) {
        *reinterpret_cast<u32x4*>(gdst) = v;
      } else {
        const OS* e = reinterpret_cast<const OS*>(&v);
#pragma unroll
        for (int t2 = 0; t2 < 16 / (int)sizeof(OS); ++t2)
          if (ncol + t2 < N) gdst[t2] = e[t2];
      }
    }
  }
}

template<class MF, class BP, class EP, int BM, int BN, int WM, int WN, int NSTAGE = 2>
int launch_core2(hipStream_t st, const void* A, int64_t lda, const typename BP::Params& bp,
                 const typename EP::Params& ep, int64_t M, int64_t N, int64_t KT,
                 int splits = 1) {
  const int m_tiles = (int)((M + BM - 1) / BM);
  const int n_tiles = (int)((N + BN - 1) / BN);
  // the stages; the epilogue stages its output panels in the same memory
  const size_t lds_bytes = NSTAGE * (size_t)(BM + BN) * kStageRow;
  auto kern = gemm_core2<MF, BP, EP, BM, BN, WM, WN, NSTAGE>;
  if (lds_bytes > 64 * 1024) {
    static std::atomic<uint64_t> lds_allowed{0};  // devices on which the kernel's LDS limit is raised
    if (!ofq_allow_dynamic_lds(reinterpret_cast<const void*>(kern), (int)lds_bytes, lds_allowed)) return OFQ_ERR_LAUNCH;
  }
  if (splits < 1 || (splits > 1 && !EP::kSplit)) return OFQ_ERR_UNSUPPORTED;
  // the copies address a tile's rows with 32-bit offsets from its first row
  if (lda * (int64_t)BM >= ((int64_t)1 << 32)) return OFQ_ERR_UNSUPPORTED;
  if constexpr (BP::kDirect) {
    if (bp.ldb * (int64_t)BN >= ((int64_t)1 << 32)) return OFQ_ERR_UNSUPPORTED;
  }
  const int kt_split = (int)((KT + splits - 1) / splits);
  if ((int64_t)kt_split * (splits - 1) >= KT) return OFQ_ERR_UNSUPPORTED;  // an empty slice
  kern<<<dim3(m_tiles * n_tiles, splits), WM * WN * 64, lds_bytes, st>>>(
      static_cast<const uint8_t*>(A), lda, bp, ep, (int)M, (int)N, (int)KT, kt_split, m_tiles,
      n_tiles);
  return ofq_check_launch();
}

}  // namespace
}  // namespace ofq
