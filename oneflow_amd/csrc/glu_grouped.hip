// The linears' neighbours in a decoder block, for groupwise-quantised weights:
//   grouped linear  -- several fused_linear_with_groupwise_quantized_weight problems in one call
//                      (the quantised counterpart of grouped_matmul_bias,
//                      oneflow/user/kernels/grouped_matmul_bias.cu:153-204: problems are grouped
//                      by shape and each group runs as one launch);
//   GLU             -- the quantised counterpart of fused_glu
//                      (oneflow/user/kernels/fused_glu_kernel.cu:303-347, :566-770):
//                      matmul_wx = x w~^T + b, matmul_vx = x v~^T + c (both stored in T),
//                      y = matmul_wx * act(matmul_vx), the activation evaluated in fp32 on the
//                      widened gate and rounded to T, the product rounded to T.
// For m <= 16 the linears of one call run as a single launch of the decode kernel; otherwise
// they run one after the other through the op's own entry point.
#include "ofq_device.h"
#include "ofq_internal.h"

namespace ofq {
namespace {

enum Activation { kActNone = 0, kActSigmoid, kActRelu, kActGelu, kActFastGelu, kActSilu };

// fp32 forms of oneflow/core/ep/common/primitive/unary_functor.h:146-170,477-484 and
// oneflow/core/ep/cuda/primitive/unary_functor.cuh:31-58 (the 16-bit types go through them:
// cuda/primitive/unary_functor.cuh:449-464,522-570)
template<int ACT>
__device__ __forceinline__ float activate(float v) {
  if constexpr (ACT == kActSigmoid) {
    return 1.0f / (1.0f + expf(-v));
  } else if constexpr (ACT == kActRelu) {
    return v <= 0.0f ? 0.0f : v;
  } else if constexpr (ACT == kActGelu) {
    return 0.5f * v * (1.0f + erff(0.70710678118654752440f * v));
  } else if constexpr (ACT == kActFastGelu) {
    const float alpha = 0.7978845608028654f;
    const float beta = 0.044714998453855515f;
    const float tanh_in = alpha * (v + beta * v * v * v);
    return 0.5f * v * (1.0f + tanhf(tanh_in));
  } else if constexpr (ACT == kActSilu) {
    return v / (1.0f + expf(-v));
  } else {
    return v;
  }
}

// y[r, c] = T( wx[r*stride + c] * T(act(vx[r*stride + c])) ), 8 elements per thread when the
// rows allow 128-bit accesses (16-bit T), else one
template<typename T, int ACT, int VEC>
__global__ void __launch_bounds__(256)
glu_forward(const typename TT<T>::storage* __restrict__ wx,
            const typename TT<T>::storage* __restrict__ vx, typename TT<T>::storage* __restrict__ y,
            int64_t m, int64_t n, int64_t stride) {
  typedef typename TT<T>::storage S;
  const int64_t per_row = n / VEC;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= m * per_row) return;
  const int64_t r = i / per_row;
  const int64_t c = (i - r * per_row) * VEC;
  S h[VEC], g[VEC], o[VEC];
  if constexpr (VEC == 8) {
    *reinterpret_cast<u32x4*>(h) = *reinterpret_cast<const u32x4*>(wx + r * stride + c);
    *reinterpret_cast<u32x4*>(g) = *reinterpret_cast<const u32x4*>(vx + r * stride + c);
  } else {
    h[0] = wx[r * stride + c];
    g[0] = vx[r * stride + c];
  }
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    const float a = TT<T>::round(activate<ACT>(TT<T>::load(&g[e])));
    TT<T>::store(&o[e], TT<T>::load(&h[e]) * a);
  }
  if constexpr (VEC == 8) {
    *reinterpret_cast<u32x4*>(y + r * n + c) = *reinterpret_cast<const u32x4*>(o);
  } else {
    y[r * n + c] = o[0];
  }
}

template<typename T, int ACT>
int launch_glu_act(hipStream_t st, const void* wx, const void* vx, void* y, int64_t m, int64_t n,
                   int64_t stride) {
  typedef typename TT<T>::storage S;
  const bool vec = sizeof(S) == 2 && n % 8 == 0 && stride % 8 == 0 && ofq_aligned16(wx)
                   && ofq_aligned16(vx) && ofq_aligned16(y);
  if (vec) {
    const int64_t threads = m * (n / 8);
    glu_forward<T, ACT, 8><<<(unsigned)((threads + 255) / 256), 256, 0, st>>>(
        static_cast<const S*>(wx), static_cast<const S*>(vx), static_cast<S*>(y), m, n, stride);
  } else {
    const int64_t threads = m * n;
    glu_forward<T, ACT, 1><<<(unsigned)((threads + 255) / 256), 256, 0, st>>>(
        static_cast<const S*>(wx), static_cast<const S*>(vx), static_cast<S*>(y), m, n, stride);
  }
  return ofq_check_launch();
}

template<typename T>
int launch_glu_t(hipStream_t st, int act, const void* wx, const void* vx, void* y, int64_t m,
                 int64_t n, int64_t stride) {
  switch (act) {
    case kActNone: return launch_glu_act<T, kActNone>(st, wx, vx, y, m, n, stride);
    case kActSigmoid: return launch_glu_act<T, kActSigmoid>(st, wx, vx, y, m, n, stride);
    case kActRelu: return launch_glu_act<T, kActRelu>(st, wx, vx, y, m, n, stride);
    case kActGelu: return launch_glu_act<T, kActGelu>(st, wx, vx, y, m, n, stride);
    case kActFastGelu: return launch_glu_act<T, kActFastGelu>(st, wx, vx, y, m, n, stride);
    case kActSilu: return launch_glu_act<T, kActSilu>(st, wx, vx, y, m, n, stride);
    default: return OFQ_ERR_BAD_ATTR;
  }
}

int launch_glu(hipStream_t st, int t_dtype, int act, const void* wx, const void* vx, void* y,
               int64_t m, int64_t n, int64_t stride) {
  switch (t_dtype) {
    case OFQ_F16: return launch_glu_t<f16>(st, act, wx, vx, y, m, n, stride);
    case OFQ_BF16: return launch_glu_t<bf16>(st, act, wx, vx, y, m, n, stride);
    case OFQ_F32: return launch_glu_t<float>(st, act, wx, vx, y, m, n, stride);
    default: return OFQ_ERR_BAD_DTYPE;
  }
}

// one problem through the op's own entry point (all of its checks apply)
int run_single(void* stream, const LinearArgs& a) {
  return ofq_fused_linear_gq(stream, a.x, a.w, a.scale, a.zero, a.bias, a.out,
                             a.w_signed ? OFQ_I8 : OFQ_U8, a.t_dtype, a.bits, a.symmetric ? 1 : 0,
                             a.group_dim, a.group_size, a.m, a.n, a.k, nullptr, 0);
}

// the argument checks of the single op that the decode kernel relies on
bool decode_args_ok(const LinearArgs& a) {
  if (a.x == nullptr || a.w == nullptr || a.scale == nullptr || a.out == nullptr) return false;
  if (a.symmetric != (a.zero == nullptr)) return false;
  if (!a.symmetric && a.w_signed) return false;
  if (a.m < 1 || a.m > 16 || a.n < 1 || a.k < 1 || a.group_size < 1) return false;
  if (a.k % a.group_size != 0) return false;
  const int64_t i32max = 0x7FFFFFFF;
  if (a.m * a.k > i32max || a.n * a.k > i32max || a.m * a.n > i32max) return false;
  return ofq_aligned16(a.x) && ofq_aligned16(a.w) && ofq_aligned16(a.scale)
         && ofq_aligned16(a.zero) && ofq_aligned16(a.bias) && ofq_aligned16(a.out);
}

// problems [begin, end) share m, k: one launch when the decode kernel takes them, else one by one
int run_group(void* stream, const LinearArgs* pr, int count) {
  hipStream_t st = static_cast<hipStream_t>(stream);
  int done = 0;
  while (done < count) {
    const int chunk = count - done < 8 ? count - done : 8;
    bool ok = chunk > 1;
    for (int i = 0; ok && i < chunk; ++i) ok = decode_args_ok(pr[done + i]);
    int rc = OFQ_ERR_UNSUPPORTED;
    if (ok) rc = launch_gemv_grouped(st, pr + done, chunk);
    if (rc == OFQ_ERR_UNSUPPORTED) {
      for (int i = 0; i < chunk; ++i) {
        rc = run_single(stream, pr[done + i]);
        if (rc != OFQ_OK) return rc;
      }
    } else if (rc != OFQ_OK) {
      return rc;
    }
    done += chunk;
  }
  return OFQ_OK;
}

}  // namespace
}  // namespace ofq

using namespace ofq;

extern "C" int ofq_grouped_linear_gq(void* stream, int count, const void* const* xs,
                                     const void* const* ws, const void* const* w_scales,
                                     const void* const* w_zeros, const void* const* bs,
                                     void* const* outs, const int64_t* ms, const int64_t* ns,
                                     const int64_t* ks, int w_dtype, int t_dtype, int num_bits,
                                     int symmetric, int group_dim, int64_t group_size) {
  OFQ_RETURN_IF(count < 0 || count > 64, OFQ_ERR_BAD_SHAPE);  // kMaxProblemBatch of the reference
  if (count == 0) return OFQ_OK;
  OFQ_RETURN_IF(xs == nullptr || ws == nullptr || w_scales == nullptr || outs == nullptr
                    || ms == nullptr || ns == nullptr || ks == nullptr,
                OFQ_ERR_NULL_POINTER);
  OFQ_RETURN_IF(w_dtype != OFQ_U8 && w_dtype != OFQ_I8, OFQ_ERR_BAD_DTYPE);
  OFQ_RETURN_IF((symmetric == 0) && w_zeros == nullptr, OFQ_ERR_NULL_POINTER);
  LinearArgs all[64];
  for (int i = 0; i < count; ++i) {
    LinearArgs& a = all[i];
    a.x = xs[i];
    a.w = ws[i];
    a.scale = w_scales[i];
    a.zero = w_zeros != nullptr ? w_zeros[i] : nullptr;
    a.bias = bs != nullptr ? bs[i] : nullptr;
    a.out = outs[i];
    a.t_dtype = t_dtype;
    a.w_signed = w_dtype == OFQ_I8;
    a.bits = num_bits;
    a.symmetric = symmetric != 0;
    a.group_dim = group_dim;
    a.group_size = group_size;
    a.m = ms[i];
    a.n = ns[i];
    a.k = ks[i];
  }
  // problems of equal (m, k) form a group, in order of first appearance
  bool taken[64] = {};
  for (int i = 0; i < count; ++i) {
    if (taken[i]) continue;
    LinearArgs grp[64];
    int gcount = 0;
    for (int j = i; j < count; ++j) {
      if (!taken[j] && all[j].m == all[i].m && all[j].k == all[i].k) {
        grp[gcount++] = all[j];
        taken[j] = true;
      }
    }
    const int rc = run_group(stream, grp, gcount);
    if (rc != OFQ_OK) return rc;
  }
  return OFQ_OK;
}

extern "C" int ofq_fused_glu_gq(void* stream, const void* x, const void* w, const void* w_scale,
                                const void* w_zero, const void* b, const void* v,
                                const void* v_scale, const void* v_zero, const void* c, void* y,
                                void* matmul_wx, void* matmul_vx, int activation, int w_dtype,
                                int t_dtype, int num_bits, int symmetric, int group_dim,
                                int64_t group_size, int64_t m, int64_t n, int64_t k) {
  OFQ_RETURN_IF(activation < kActNone || activation > kActSilu, OFQ_ERR_BAD_ATTR);
  OFQ_RETURN_IF(m < 0 || n < 0 || k <= 0, OFQ_ERR_BAD_SHAPE);
  OFQ_RETURN_IF(w_dtype != OFQ_U8 && w_dtype != OFQ_I8, OFQ_ERR_BAD_DTYPE);
  if (m == 0 || n == 0) return OFQ_OK;
  OFQ_RETURN_IF(y == nullptr || matmul_wx == nullptr, OFQ_ERR_NULL_POINTER);
  const bool split = v != nullptr;
  // expected existence of c only with b, and of both in split mode
  // (oneflow/core/functional/impl/nn_functor.cpp:3736-3746)
  OFQ_RETURN_IF(b == nullptr && c != nullptr, OFQ_ERR_NULL_POINTER);
  OFQ_RETURN_IF(split && b != nullptr && c == nullptr, OFQ_ERR_NULL_POINTER);
  OFQ_RETURN_IF(split && (matmul_vx == nullptr || v_scale == nullptr), OFQ_ERR_NULL_POINTER);
  hipStream_t st = static_cast<hipStream_t>(stream);
  LinearArgs a[2];
  a[0].x = x;
  a[0].w = w;
  a[0].scale = w_scale;
  a[0].zero = w_zero;
  a[0].bias = b;
  a[0].out = matmul_wx;
  a[0].t_dtype = t_dtype;
  a[0].w_signed = w_dtype == OFQ_I8;
  a[0].bits = num_bits;
  a[0].symmetric = symmetric != 0;
  a[0].group_dim = group_dim;
  a[0].group_size = group_size;
  a[0].m = m;
  a[0].n = split ? n : 2 * n;  // one weight of 2n rows: hidden state first, gate second
  a[0].k = k;
  int rc;
  if (split) {
    a[1] = a[0];
    a[1].w = v;
    a[1].scale = v_scale;
    a[1].zero = v_zero;
    a[1].bias = c;
    a[1].out = matmul_vx;
    // decode, fp16, 4-bit codes: both linears and the gating as one launch
    if (m <= 16 && t_dtype == OFQ_F16 && decode_args_ok(a[0]) && decode_args_ok(a[1])
        && ofq_aligned16(y)) {
      rc = launch_gemv_glu(st, a[0], a[1], y, activation);
      if (rc != OFQ_ERR_UNSUPPORTED) return rc;
    }
    rc = run_group(stream, a, 2);
  } else {
    rc = run_single(stream, a[0]);
  }
  if (rc != OFQ_OK) return rc;
  const size_t esz = t_dtype == OFQ_F32 ? 4 : 2;
  const void* gate = split ? matmul_vx
                           : static_cast<const void*>(static_cast<const char*>(matmul_wx) + n * esz);
  return launch_glu(st, t_dtype, activation, matmul_wx, gate, y, m, n, split ? n : 2 * n);
}
