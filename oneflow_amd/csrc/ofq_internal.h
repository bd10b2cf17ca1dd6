// Launchers shared between translation units of the library (not part of the C ABI).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ofq {

struct LinearArgs {
  const void* x;        // [m,k] T
  const void* w;        // [n, k*bits/8] bytes
  const void* scale;    // [n, k/group_size] T
  const void* zero;     // same or nullptr
  const void* bias;     // [n] T or nullptr
  void* out;            // [m,n] T
  int t_dtype;          // OFQ_F16 | OFQ_BF16 | OFQ_F32
  bool w_signed;        // int8 container
  int bits;             // 4 | 8
  bool symmetric;
  int group_dim;        // 0 | 1
  int64_t group_size;
  int64_t m, n, k;
};

// MFMA GEMM with in-tile dequantisation; groups along K.  Returns OFQ_ERR_UNSUPPORTED when the
// shape does not meet the kernel's tiling constraints (caller falls back).
// With a workspace of gemm_wq_workspace_bytes() (non-zero for large m only) the weight is
// dequantised once into it and a copy-fed GEMM runs on the result; without one the in-tile path
// is used.
bool gemm_wq_supported(const LinearArgs& a);
size_t gemm_wq_workspace_bytes(const LinearArgs& a);
int launch_gemm_wq(hipStream_t st, const LinearArgs& a, void* workspace, size_t workspace_bytes);

// m = 1, fp16, 4-bit symmetric codes in an int8 container, groups along K: a wave owns whole
// weight rows (contiguous requests, packed dot products, no cross-wave fold).
bool gemv_m1_supported(const LinearArgs& a);
int launch_gemv_m1(hipStream_t st, const LinearArgs& a);
int launch_gemv_m1_grouped(hipStream_t st, const LinearArgs* problems, int count);
int launch_gemv_m1_glu(hipStream_t st, const LinearArgs& a, const LinearArgs& g, void* y, int act);
// the same for groups along N (scale [n / group_size, k]): the scale meets x, once per block
bool gemv_m1_gn_supported(const LinearArgs& a);
int launch_gemv_m1_gn(hipStream_t st, const LinearArgs& a);

// m = 1, fp16 or bf16, 4- or 8-bit codes in either container, symmetric or with a zero point,
// groups along K of a power-of-two size: the same row-per-wave structure with the reference's
// roundings of w~.
bool gemv_m1_any_supported(const LinearArgs& a);
int launch_gemv_m1_any(hipStream_t st, const LinearArgs& a);

// Skinny-M (m <= 16) MFMA GEMV that streams the weights once.
bool gemv_wq_supported(const LinearArgs& a);
int launch_gemv_wq(hipStream_t st, const LinearArgs& a);

// 16 < m <= 64 without a workspace: the decode kernel's row split with several 16-row tiles of x
// per weight tile.
bool gemv_mt_supported(const LinearArgs& a);
int launch_gemv_mt(hipStream_t st, const LinearArgs& a);

// Groups along N (group_dim = 0), fp16 / bf16: the streaming kernel with one scale per k (any m,
// 64 rows of x per pass over the weights), and for m > 64 with a workspace of
// gemm_gn_workspace_bytes() the weight dequantised once plus a copy-fed GEMM.
bool gemv_gn_supported(const LinearArgs& a);
int launch_gemv_gn(hipStream_t st, const LinearArgs& a);
size_t gemm_gn_workspace_bytes(const LinearArgs& a);
int launch_gemm_gn(hipStream_t st, const LinearArgs& a, void* workspace);

// Up to 8 decode linears that share m, k, dtype and quantisation attributes (x, w, scale, zero,
// bias, out and n per problem) as ONE launch of the natural-order decode kernel.
// OFQ_ERR_UNSUPPORTED when the shapes do not fit it (caller launches the problems one by one).
int launch_gemv_grouped(hipStream_t st, const LinearArgs* problems, int count);

// fused_glu in split mode for decode: hidden = x w~^T + b -> a.out, gate = x v~^T + c -> g.out,
// y = hidden * act(gate), all in ONE launch (every block owns the same rows of both weights).
// a and g differ in w / scale / zero / bias / out only.  OFQ_ERR_UNSUPPORTED when the shapes do
// not fit (caller runs the linears and the gating separately).
int launch_gemv_glu(hipStream_t st, const LinearArgs& a, const LinearArgs& g, void* y, int act);

// matmul_quant with few rows of a: int8 MFMA with the weights streamed once, 64 rows of a per
// pass (any m; k a multiple of 64).
bool matmul_quant_rows_supported(int64_t m, int64_t n, int64_t k);
int launch_matmul_quant_rows(hipStream_t st, const void* a, const void* b, const float* a_scale,
                             const float* b_scale, const void* bias, void* out, int out_dtype,
                             int64_t m, int64_t n, int64_t k);

// Any shape / grouping; one wave per output element.
int launch_linear_generic(hipStream_t st, const LinearArgs& a);

}  // namespace ofq
