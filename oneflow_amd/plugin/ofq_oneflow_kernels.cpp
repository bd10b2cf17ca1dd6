// OneFlow user-op kernels for the quantized-inference family, backed by the HIP library behind
// include/ofq.h.  This file is the C++ host side of the drop-in: it registers kernels under the
// reference's op names and argument names and forwards to the C ABI.  It is written against
// OneFlow's user-op API (oneflow/core/framework/framework.h); with -DOFQ_PLUGIN_STANDALONE it
// compiles against the minimal restatement in standalone/ so that the registrations can be
// exercised without a OneFlow build.
//
// Replaced registrations (device kCUDA, the only accelerator value of DeviceType,
// oneflow/core/common/device_type.proto:4-13):
//   groupwise_dequantize                          groupwise_quantization_kernels.cu:456-463
//   fused_linear_with_groupwise_quantized_weight  groupwise_quantization_kernels.cu:844-851
//   min_max_observer                              min_max_observer_kernel.cu:240-258
//   moving_average_min_max_observer               moving_average_min_max_observer_kernel.cu:306-314
//   quantization                                  quantization_kernel.cu:149-156
//   fake_quantization                             fake_quantization_kernel.cu:150-157
// Added registrations (ops without a kernel in the reference tree; their op definitions would sit
// next to OneFlowUserOps.td:8248-8387 with the argument names used here):
//   fused_layer_norm_min_max_observer      x, [gamma], [beta], [bias], [skip] -> y, scale, zero_point
//   fused_layer_norm_quantization          x, [gamma], [beta] -> out (int8), scale, zero_point
//   matmul_quant                           a, b, a_scale, b_scale, [bias] -> out
//   fused_glu_with_groupwise_quantized_weight      arguments of fused_glu + the weights' scales / zeros
//   grouped_linear_with_groupwise_quantized_weight variadic xs, ws, w_scales, [w_zeros], [bs] -> ys
// bf16 variants are added; kernels carry kKernelPriorityOptimized so that they win over stock
// kernels registered for the same (op, device, dtype)
// (oneflow/core/framework/user_op_registry_manager.cpp:95-114).
#include "oneflow/core/framework/framework.h"
#include "oneflow/core/ep/cuda/cuda_stream.h"
#include "oneflow/core/kernel/cuda_graph_support.h"

#include "ofq.h"
#include "ofq_hip_shim.h"

namespace oneflow {

namespace {

// OneFlow hands out the raw device stream through ep::CudaStream::cuda_stream()
// (oneflow/core/ep/cuda/cuda_stream.h:91, the call of groupwise_quantization_kernels.cu:531); on
// this device that handle IS the hipStream_t: ep_hip/oneflow/core/ep/cuda/cuda_stream.{h,cpp} is
// ep::CudaStream over a HIP stream, under the reference's include path and spelling, so this
// source is one text for a OneFlow tree and for the stand-alone build.
inline void* RawStream(user_op::KernelComputeContext* ctx) {
  return ctx->stream()->As<ep::CudaStream>()->cuda_stream();
}

inline int ToOfq(DataType dt) {
  switch (dt) {
    case DataType::kFloat: return OFQ_F32;
    case DataType::kFloat16: return OFQ_F16;
    case DataType::kBFloat16: return OFQ_BF16;
    case DataType::kDouble: return OFQ_F64;
    case DataType::kInt8: return OFQ_I8;
    case DataType::kUInt8: return OFQ_U8;
    default: UNIMPLEMENTED(); return -1;
  }
}

// Argument errors end the process like the CHECKs of the kernels these replace.  A failed launch
// does not: the reference's kernels do not test their launches either, the runtime asks the
// stream after Compute (CHECK_JUST(stream->GetAsyncError()), stateful_opkernel.cpp:1007), and the
// library keeps the device runtime's error for that query.
inline void CheckOk(int status, const char* what) {
  if (status != OFQ_OK && status != OFQ_ERR_LAUNCH) {
    std::cerr << what << ": " << ofq_status_string(status) << "\n";
    CHECK_EQ(status, OFQ_OK);
  }
}

inline int Scheme(const std::string& s) {
  return s == "symmetric" ? OFQ_SCHEME_SYMMETRIC : OFQ_SCHEME_AFFINE;
}
inline int Formula(const std::string& s) {
  return s == "google" ? OFQ_FORMULA_GOOGLE : OFQ_FORMULA_CAMBRICON;
}

}  // namespace

// ---- groupwise_dequantize: args in, scale, [zero] -> out; attrs num_bits, symmetric,
//      group_dim, group_size (OneFlowUserOps.td:8343-8362) ------------------------------------
class OfqGroupwiseDequantizeKernel final : public user_op::OpKernel,
                                           public user_op::CudaGraphSupport {
 public:
  using user_op::OpKernel::Compute;
  void Compute(user_op::KernelComputeContext* ctx) const override {
    const user_op::Tensor* in = ctx->Tensor4ArgNameAndIndex("in", 0);
    const user_op::Tensor* scale = ctx->Tensor4ArgNameAndIndex("scale", 0);
    const user_op::Tensor* zero =
        ctx->has_input("zero", 0) ? ctx->Tensor4ArgNameAndIndex("zero", 0) : nullptr;
    user_op::Tensor* out = ctx->Tensor4ArgNameAndIndex("out", 0);
    const int64_t group_size = ctx->Attr<int64_t>("group_size");
    const int64_t group_dim = ctx->Attr<int64_t>("group_dim");
    const int32_t num_bits = ctx->Attr<int32_t>("num_bits");
    const bool symmetric = ctx->Attr<bool>("symmetric");
    // shape rules of GroupwiseDequantizeKernel::Compute, groupwise_quantization_kernels.cu:409-437
    const int64_t axes = in->shape_view().NumAxes();
    CHECK_GE(axes, 1);
    CHECK_EQ(scale->shape_view().NumAxes(), axes);
    CHECK_EQ(out->shape_view().NumAxes(), axes);
    CHECK_GE(group_dim, 0);
    CHECK_LT(group_dim, axes);
    for (int64_t i = 0; i < axes; ++i) {
      const int64_t f = (i == axes - 1) ? 8 / num_bits : 1;
      CHECK_EQ(out->shape_view().At(i), in->shape_view().At(i) * f);
    }
    const int64_t group_dim_size = out->shape_view().At(group_dim);
    CHECK_GT(group_size, 0);
    CHECK_LE(group_size, group_dim_size);
    CHECK_EQ(group_dim_size % group_size, 0);
    const int64_t num_groups = group_dim_size / group_size;
    for (int64_t i = 0; i < axes; ++i) {
      const int64_t expected = i == group_dim ? num_groups : out->shape_view().At(i);
      CHECK_EQ(scale->shape_view().At(i), expected);
      if (zero != nullptr) { CHECK_EQ(zero->shape_view().At(i), expected); }
    }
    const int64_t outer = out->shape_view().Count(0, group_dim) * num_groups;
    const int64_t inner = out->shape_view().Count(group_dim + 1);
    CheckOk(ofq_groupwise_dequantize(RawStream(ctx), in->dptr(), scale->dptr(),
                                     zero ? zero->dptr() : nullptr, out->mut_dptr(),
                                     ToOfq(in->data_type()), ToOfq(scale->data_type()), num_bits,
                                     symmetric ? 1 : 0, outer, group_size, inner),
            "groupwise_dequantize");
  }
  bool AlwaysComputeWhenAllOutputsEmpty() const override { return false; }
};

#define REGISTER_OFQ_DEQUANTIZE(dtype)                                       \
  REGISTER_USER_KERNEL("groupwise_dequantize")                               \
      .SetCreateFn<OfqGroupwiseDequantizeKernel>()                           \
      .SetIsMatchedHob((user_op::HobDeviceType() == DeviceType::kCUDA)       \
                       && (user_op::HobDataType("scale", 0) == dtype))       \
      .SetPriority(user_op::kKernelPriorityOptimized)
REGISTER_OFQ_DEQUANTIZE(DataType::kFloat16);
REGISTER_OFQ_DEQUANTIZE(DataType::kBFloat16);
REGISTER_OFQ_DEQUANTIZE(DataType::kFloat);

// ---- fused_linear_with_groupwise_quantized_weight: x, w, w_scale, [w_zero], [b] -> out -----
class OfqFusedLinearKernel final : public user_op::OpKernel, public user_op::CudaGraphSupport {
 public:
  using user_op::OpKernel::Compute;
  void Compute(user_op::KernelComputeContext* ctx, user_op::OpKernelState*,
               const user_op::OpKernelCache*) const override {
    const user_op::Tensor* x = ctx->Tensor4ArgNameAndIndex("x", 0);
    const user_op::Tensor* w = ctx->Tensor4ArgNameAndIndex("w", 0);
    const user_op::Tensor* w_scale = ctx->Tensor4ArgNameAndIndex("w_scale", 0);
    const user_op::Tensor* b = ctx->has_input("b", 0) ? ctx->Tensor4ArgNameAndIndex("b", 0) : nullptr;
    const user_op::Tensor* w_zero =
        ctx->has_input("w_zero", 0) ? ctx->Tensor4ArgNameAndIndex("w_zero", 0) : nullptr;
    user_op::Tensor* out = ctx->Tensor4ArgNameAndIndex("out", 0);
    const DataType data_type = x->data_type();
    CHECK_EQ(w_scale->data_type(), data_type);
    CHECK_EQ(out->data_type(), data_type);
    const int64_t group_size = ctx->Attr<int64_t>("group_size");
    const int64_t group_dim = ctx->Attr<int64_t>("group_dim");
    const int32_t num_bits = ctx->Attr<int32_t>("num_bits");
    const bool symmetric = ctx->Attr<bool>("symmetric");
    // shape rules of the reference kernel, groupwise_quantization_kernels.cu:778-822
    CHECK_GE(x->shape_view().NumAxes(), 2);
    const int64_t k = x->shape_view().At(x->shape_view().NumAxes() - 1);
    const int64_t m = x->shape_view().elem_cnt() / k;
    CHECK_EQ(w->shape_view().NumAxes(), 2);
    CHECK_EQ(w->shape_view().At(1) * (8 / num_bits), k);
    const int64_t n = w->shape_view().At(0);
    const int64_t num_groups = (group_dim == 0 ? n : k) / group_size;
    CHECK_EQ(w_scale->shape_view().At(0), group_dim == 0 ? num_groups : n);
    CHECK_EQ(w_scale->shape_view().At(1), group_dim == 0 ? k : num_groups);
    if (w_zero != nullptr) { CHECK(w_zero->shape_view() == w_scale->shape_view()); }
    if (b != nullptr) { CHECK_EQ(b->shape_view().At(0), n); }
    CHECK_EQ(out->shape_view().At(out->shape_view().NumAxes() - 1), n);
    CHECK_EQ(symmetric, w_zero == nullptr);
    // tmp_buffer exists when the InferTmpSizeFn below asked for one (large m: the weight is
    // dequantised once into it and a copy-fed GEMM runs on the result)
    user_op::Tensor* tmp = ctx->Tensor4ArgNameAndIndex("tmp_buffer", 0);
    CheckOk(ofq_fused_linear_gq(RawStream(ctx), x->dptr(), w->dptr(), w_scale->dptr(),
                                w_zero ? w_zero->dptr() : nullptr, b ? b->dptr() : nullptr,
                                out->mut_dptr(), ToOfq(w->data_type()), ToOfq(data_type), num_bits,
                                symmetric ? 1 : 0, (int)group_dim, group_size, m, n, k,
                                tmp ? tmp->mut_dptr() : nullptr,
                                tmp ? (size_t)tmp->shape_view().elem_cnt() : 0),
            "fused_linear_with_groupwise_quantized_weight");
  }
  bool AlwaysComputeWhenAllOutputsEmpty() const override { return false; }
};

#define REGISTER_OFQ_FUSED_LINEAR(dtype)                                     \
  REGISTER_USER_KERNEL("fused_linear_with_groupwise_quantized_weight")       \
      .SetCreateFn<OfqFusedLinearKernel>()                                   \
      .SetIsMatchedHob((user_op::HobDeviceType() == DeviceType::kCUDA)       \
                       && (user_op::HobDataType("out", 0) == dtype))         \
      .SetInferTmpSizeFn([](user_op::InferContext* ctx) -> size_t {          \
        const ShapeView xs = ctx->InputShape("x", 0);                        \
        const ShapeView ws = ctx->InputShape("w", 0);                        \
        const int64_t k = xs.At(xs.NumAxes() - 1);                           \
        return ofq_fused_linear_gq_workspace_bytes(                          \
            ToOfq(ctx->InputDType("w", 0)), ToOfq(dtype),                    \
            ctx->Attr<int32_t>("num_bits"), ctx->Attr<bool>("symmetric"),    \
            (int)ctx->Attr<int64_t>("group_dim"),                            \
            ctx->Attr<int64_t>("group_size"), xs.elem_cnt() / k, ws.At(0),   \
            k);                                                              \
      })                                                                     \
      .SetPriority(user_op::kKernelPriorityOptimized)
REGISTER_OFQ_FUSED_LINEAR(DataType::kFloat16);
REGISTER_OFQ_FUSED_LINEAR(DataType::kBFloat16);
REGISTER_OFQ_FUSED_LINEAR(DataType::kFloat);

// ---- min_max_observer: in -> scale, zero_point (+ tmp_buffer) -------------------------------
class OfqMinMaxObserverKernel final : public user_op::OpKernel {
 public:
  using user_op::OpKernel::Compute;
  void Compute(user_op::KernelComputeContext* ctx) const override {
    const user_op::Tensor* in = ctx->Tensor4ArgNameAndIndex("in", 0);
    user_op::Tensor* scale = ctx->Tensor4ArgNameAndIndex("scale", 0);
    user_op::Tensor* zero_point = ctx->Tensor4ArgNameAndIndex("zero_point", 0);
    user_op::Tensor* tmp = ctx->Tensor4ArgNameAndIndex("tmp_buffer", 0);
    const bool per_layer = ctx->Attr<bool>("per_layer_quantization");
    const int64_t elem_cnt = in->shape_view().elem_cnt();
    const int64_t channels = per_layer ? 1 : in->shape_view().At(0);
    CheckOk(ofq_min_max_observer(RawStream(ctx), in->dptr(), scale->mut_dptr(),
                                 zero_point->mut_dptr(), ToOfq(in->data_type()), elem_cnt, channels,
                                 ctx->Attr<int32_t>("quantization_bit"),
                                 Scheme(ctx->Attr<std::string>("quantization_scheme")),
                                 Formula(ctx->Attr<std::string>("quantization_formula")),
                                 tmp->mut_dptr(), (size_t)tmp->shape_view().elem_cnt()),
            "min_max_observer");
  }
  bool AlwaysComputeWhenAllOutputsEmpty() const override { return false; }
};

#define REGISTER_OFQ_OBSERVER(dtype)                                                         \
  REGISTER_USER_KERNEL("min_max_observer")                                                   \
      .SetCreateFn<OfqMinMaxObserverKernel>()                                                \
      .SetIsMatchedHob((user_op::HobDeviceType() == DeviceType::kCUDA)                       \
                       && (user_op::HobDataType("in", 0) == dtype))                          \
      .SetInferTmpSizeFn([](user_op::InferContext* ctx) -> size_t {                          \
        const ShapeView shape = ctx->InputShape("in", 0);                                    \
        const int64_t channels = ctx->Attr<bool>("per_layer_quantization") ? 1 : shape.At(0);\
        return ofq_min_max_observer_workspace_bytes(dtype == DataType::kDouble ? OFQ_F64     \
                                                                               : OFQ_F32,    \
                                                    shape.elem_cnt(), channels);             \
      })                                                                                     \
      .SetPriority(user_op::kKernelPriorityOptimized)
REGISTER_OFQ_OBSERVER(DataType::kFloat);
REGISTER_OFQ_OBSERVER(DataType::kDouble);

// ---- moving_average_min_max_observer: in, current_train_step, moving_max, moving_min ->
//      scale, zero_point (+ tmp_buffer); moving_* are updated in place ------------------------
class OfqMovingAverageMinMaxObserverKernel final : public user_op::OpKernel {
 public:
  using user_op::OpKernel::Compute;
  void Compute(user_op::KernelComputeContext* ctx) const override {
    const user_op::Tensor* in = ctx->Tensor4ArgNameAndIndex("in", 0);
    const user_op::Tensor* step = ctx->Tensor4ArgNameAndIndex("current_train_step", 0);
    user_op::Tensor* moving_max = ctx->Tensor4ArgNameAndIndex("moving_max", 0);
    user_op::Tensor* moving_min = ctx->Tensor4ArgNameAndIndex("moving_min", 0);
    user_op::Tensor* scale = ctx->Tensor4ArgNameAndIndex("scale", 0);
    user_op::Tensor* zero_point = ctx->Tensor4ArgNameAndIndex("zero_point", 0);
    user_op::Tensor* tmp = ctx->Tensor4ArgNameAndIndex("tmp_buffer", 0);
    CheckOk(ofq_moving_average_min_max_observer(
                RawStream(ctx), in->dptr(), static_cast<const int64_t*>(step->dptr()),
                moving_max->mut_dptr(), moving_min->mut_dptr(), scale->mut_dptr(),
                zero_point->mut_dptr(), ToOfq(in->data_type()), in->shape_view().elem_cnt(),
                ctx->Attr<int32_t>("quantization_bit"),
                Scheme(ctx->Attr<std::string>("quantization_scheme")),
                Formula(ctx->Attr<std::string>("quantization_formula")),
                ctx->Attr<float>("momentum"), ctx->Attr<int64_t>("stop_update_after_iters"),
                ctx->Attr<bool>("training") ? 1 : 0, tmp->mut_dptr(),
                (size_t)tmp->shape_view().elem_cnt()),
            "moving_average_min_max_observer");
  }
  bool AlwaysComputeWhenAllOutputsEmpty() const override { return false; }
};

#define REGISTER_OFQ_MOVING_OBSERVER(dtype)                                                  \
  REGISTER_USER_KERNEL("moving_average_min_max_observer")                                    \
      .SetCreateFn<OfqMovingAverageMinMaxObserverKernel>()                                   \
      .SetIsMatchedHob((user_op::HobDeviceType() == DeviceType::kCUDA)                       \
                       && (user_op::HobDataType("in", 0) == dtype))                          \
      .SetInferTmpSizeFn([](user_op::InferContext* ctx) -> size_t {                          \
        return ofq_moving_average_min_max_observer_workspace_bytes(                          \
            dtype == DataType::kDouble ? OFQ_F64 : OFQ_F32,                                  \
            ctx->InputShape("in", 0).elem_cnt());                                            \
      })                                                                                     \
      .SetPriority(user_op::kKernelPriorityOptimized)
REGISTER_OFQ_MOVING_OBSERVER(DataType::kFloat);
REGISTER_OFQ_MOVING_OBSERVER(DataType::kDouble);

// ---- quantization / fake_quantization: in, scale, zero_point -> out ---------------------------
template<bool kFake>
class OfqQuantizationKernel final : public user_op::OpKernel {
 public:
  using user_op::OpKernel::Compute;
  void Compute(user_op::KernelComputeContext* ctx) const override {
    const user_op::Tensor* in = ctx->Tensor4ArgNameAndIndex("in", 0);
    const user_op::Tensor* scale = ctx->Tensor4ArgNameAndIndex("scale", 0);
    const user_op::Tensor* zero_point = ctx->Tensor4ArgNameAndIndex("zero_point", 0);
    user_op::Tensor* out = ctx->Tensor4ArgNameAndIndex("out", 0);
    const int64_t elem_cnt = in->shape_view().elem_cnt();
    const int64_t scale_size = scale->shape_view().elem_cnt();
    const int bits = ctx->Attr<int32_t>("quantization_bit");
    const int scheme = Scheme(ctx->Attr<std::string>("quantization_scheme"));
    const int formula = Formula(ctx->Attr<std::string>("quantization_formula"));
    const int dt = ToOfq(in->data_type());
    // OFQ_ZP_FLOAT: the zero-point rule of the CUDA kernels this replaces
    if (kFake) {
      CheckOk(ofq_fake_quantization(RawStream(ctx), in->dptr(), scale->dptr(), zero_point->dptr(),
                                    out->mut_dptr(), dt, elem_cnt, scale_size, bits, scheme,
                                    formula, OFQ_ZP_FLOAT),
              "fake_quantization");
    } else {
      CheckOk(ofq_quantization(RawStream(ctx), in->dptr(), scale->dptr(), zero_point->dptr(),
                               out->mut_dptr(), dt, dt, elem_cnt, scale_size, bits, scheme,
                               formula, OFQ_ZP_FLOAT),
              "quantization");
    }
  }
  bool AlwaysComputeWhenAllOutputsEmpty() const override { return false; }
};

#define REGISTER_OFQ_QUANTIZATION(op_name, fake, dtype)                      \
  REGISTER_USER_KERNEL(op_name)                                              \
      .SetCreateFn<OfqQuantizationKernel<fake>>()                            \
      .SetIsMatchedHob((user_op::HobDeviceType() == DeviceType::kCUDA)       \
                       && (user_op::HobDataType("in", 0) == dtype))          \
      .SetPriority(user_op::kKernelPriorityOptimized)
REGISTER_OFQ_QUANTIZATION("quantization", false, DataType::kFloat);
REGISTER_OFQ_QUANTIZATION("quantization", false, DataType::kDouble);
REGISTER_OFQ_QUANTIZATION("fake_quantization", true, DataType::kFloat);
REGISTER_OFQ_QUANTIZATION("fake_quantization", true, DataType::kDouble);

// ---- fused_layer_norm_min_max_observer: x, [gamma], [beta], [bias], [skip] -> y, scale,
//      zero_point (+ tmp_buffer); attrs epsilon, alpha (double), quantization_bit.  With bias /
//      skip the normalised row is that of skip_layer_norm (skip_layer_norm_kernel.cu:36-67). ----
class OfqLayerNormObserverKernel final : public user_op::OpKernel, public user_op::CudaGraphSupport {
 public:
  using user_op::OpKernel::Compute;
  void Compute(user_op::KernelComputeContext* ctx, user_op::OpKernelState*,
               const user_op::OpKernelCache*) const override {
    auto opt = [&](const char* name) -> const user_op::Tensor* {
      return ctx->has_input(name, 0) ? ctx->Tensor4ArgNameAndIndex(name, 0) : nullptr;
    };
    const user_op::Tensor* x = ctx->Tensor4ArgNameAndIndex("x", 0);
    const user_op::Tensor* gamma = opt("gamma");
    const user_op::Tensor* beta = opt("beta");
    const user_op::Tensor* bias = opt("bias");
    const user_op::Tensor* skip = opt("skip");
    user_op::Tensor* y = ctx->Tensor4ArgNameAndIndex("y", 0);
    user_op::Tensor* scale = ctx->Tensor4ArgNameAndIndex("scale", 0);
    user_op::Tensor* zero_point = ctx->Tensor4ArgNameAndIndex("zero_point", 0);
    user_op::Tensor* tmp = ctx->Tensor4ArgNameAndIndex("tmp_buffer", 0);
    CHECK_GE(x->shape_view().NumAxes(), 2);
    const int64_t cols = x->shape_view().At(x->shape_view().NumAxes() - 1);
    const int64_t rows = x->shape_view().elem_cnt() / cols;
    if (gamma != nullptr) { CHECK_EQ(gamma->shape_view().elem_cnt(), cols); }
    if (beta != nullptr) { CHECK_EQ(beta->shape_view().elem_cnt(), cols); }
    if (bias != nullptr) { CHECK_EQ(bias->shape_view().elem_cnt(), cols); }
    if (skip != nullptr) { CHECK(skip->shape_view() == x->shape_view()); }
    CHECK_EQ(scale->data_type(), DataType::kFloat);
    CHECK(tmp != nullptr);
    const size_t tmp_bytes = (size_t)tmp->shape_view().elem_cnt();
    const int dt = ToOfq(x->data_type());
    if (bias != nullptr || skip != nullptr) {
      CheckOk(ofq_fused_skip_layer_norm_min_max_observer(
                  RawStream(ctx), x->dptr(), bias ? bias->dptr() : nullptr,
                  skip ? skip->dptr() : nullptr, ctx->Attr<double>("alpha"),
                  gamma ? gamma->dptr() : nullptr, beta ? beta->dptr() : nullptr, y->mut_dptr(),
                  scale->mut_dptr<float>(), zero_point->mut_dptr<float>(), dt, rows, cols,
                  ctx->Attr<double>("epsilon"), ctx->Attr<int32_t>("quantization_bit"),
                  tmp->mut_dptr(), tmp_bytes),
              "fused_skip_layer_norm_min_max_observer");
    } else {
      CheckOk(ofq_fused_layer_norm_min_max_observer(
                  RawStream(ctx), x->dptr(), gamma ? gamma->dptr() : nullptr,
                  beta ? beta->dptr() : nullptr, y->mut_dptr(), scale->mut_dptr<float>(),
                  zero_point->mut_dptr<float>(), dt, rows, cols, ctx->Attr<double>("epsilon"),
                  ctx->Attr<int32_t>("quantization_bit"), tmp->mut_dptr(), tmp_bytes),
              "fused_layer_norm_min_max_observer");
    }
  }
  bool AlwaysComputeWhenAllOutputsEmpty() const override { return false; }
};

#define REGISTER_OFQ_LN_OBSERVER(dtype)                                                       \
  REGISTER_USER_KERNEL("fused_layer_norm_min_max_observer")                                   \
      .SetCreateFn<OfqLayerNormObserverKernel>()                                              \
      .SetIsMatchedHob((user_op::HobDeviceType() == DeviceType::kCUDA)                        \
                       && (user_op::HobDataType("y", 0) == dtype))                            \
      .SetInferTmpSizeFn([](user_op::InferContext* ctx) -> size_t {                           \
        const ShapeView xs = ctx->InputShape("x", 0);                                         \
        const int64_t cols = xs.At(xs.NumAxes() - 1);                                         \
        return ofq_fused_layer_norm_min_max_observer_workspace_bytes(ToOfq(dtype),            \
                                                                     xs.elem_cnt() / cols,    \
                                                                     cols);                   \
      })                                                                                      \
      .SetPriority(user_op::kKernelPriorityOptimized)
REGISTER_OFQ_LN_OBSERVER(DataType::kFloat16);
REGISTER_OFQ_LN_OBSERVER(DataType::kBFloat16);
REGISTER_OFQ_LN_OBSERVER(DataType::kFloat);

// ---- fused_layer_norm_quantization: x, [gamma], [beta] -> out (int8 codes), scale, zero_point;
//      attrs epsilon (double), quantization_bit (int32): fused_layer_norm_min_max_observer followed
//      by quantization (symmetric, per layer) of its y.  The library serves the register-resident
//      shapes with two kernels that never write y; for every other shape this kernel runs the two
//      ops itself, y in the op's tmp_buffer -- the same bits either way -------------------------
inline size_t LnQuantYBytes(DataType dtype, int64_t rows, int64_t cols) {
  const size_t elem = dtype == DataType::kFloat ? 4 : 2;
  return ((size_t)rows * (size_t)cols * elem + 255) & ~(size_t)255;
}
inline size_t LnQuantTmpBytes(DataType dtype, int64_t rows, int64_t cols) {
  const size_t fused = ofq_fused_layer_norm_quantization_workspace_bytes(ToOfq(dtype), rows, cols);
  const size_t two_ops = LnQuantYBytes(dtype, rows, cols)
                         + ofq_fused_layer_norm_min_max_observer_workspace_bytes(ToOfq(dtype), rows,
                                                                                 cols);
  return fused > two_ops ? fused : two_ops;
}
class OfqLayerNormQuantizationKernel final : public user_op::OpKernel,
                                             public user_op::CudaGraphSupport {
 public:
  using user_op::OpKernel::Compute;
  void Compute(user_op::KernelComputeContext* ctx, user_op::OpKernelState*,
               const user_op::OpKernelCache*) const override {
    const user_op::Tensor* x = ctx->Tensor4ArgNameAndIndex("x", 0);
    const user_op::Tensor* gamma =
        ctx->has_input("gamma", 0) ? ctx->Tensor4ArgNameAndIndex("gamma", 0) : nullptr;
    const user_op::Tensor* beta =
        ctx->has_input("beta", 0) ? ctx->Tensor4ArgNameAndIndex("beta", 0) : nullptr;
    user_op::Tensor* out = ctx->Tensor4ArgNameAndIndex("out", 0);
    user_op::Tensor* scale = ctx->Tensor4ArgNameAndIndex("scale", 0);
    user_op::Tensor* zero_point = ctx->Tensor4ArgNameAndIndex("zero_point", 0);
    user_op::Tensor* tmp = ctx->Tensor4ArgNameAndIndex("tmp_buffer", 0);
    CHECK_GE(x->shape_view().NumAxes(), 2);
    const int64_t cols = x->shape_view().At(x->shape_view().NumAxes() - 1);
    const int64_t rows = x->shape_view().elem_cnt() / cols;
    if (gamma != nullptr) { CHECK_EQ(gamma->shape_view().elem_cnt(), cols); }
    if (beta != nullptr) { CHECK_EQ(beta->shape_view().elem_cnt(), cols); }
    CHECK_EQ(out->data_type(), DataType::kInt8);
    CHECK_EQ(scale->data_type(), DataType::kFloat);
    CHECK(tmp != nullptr);
    const size_t tmp_bytes = (size_t)tmp->shape_view().elem_cnt();
    CHECK_GE(tmp_bytes, LnQuantTmpBytes(x->data_type(), rows, cols));
    const int dt = ToOfq(x->data_type());
    const double epsilon = ctx->Attr<double>("epsilon");
    const int32_t bits = ctx->Attr<int32_t>("quantization_bit");
    const int status = ofq_fused_layer_norm_quantization(
        RawStream(ctx), x->dptr(), gamma ? gamma->dptr() : nullptr, beta ? beta->dptr() : nullptr,
        out->mut_dptr(), scale->mut_dptr<float>(), zero_point->mut_dptr<float>(), dt, rows, cols,
        epsilon, bits, OFQ_LN_STATS_FP32, tmp->mut_dptr(), tmp_bytes);
    if (status != OFQ_ERR_UNSUPPORTED) {
      CheckOk(status, "fused_layer_norm_quantization");
      return;
    }
    // the two ops: y at the front of tmp_buffer, the observer's partial maxima behind it
    char* y = tmp->mut_dptr<char>();
    const size_t y_bytes = LnQuantYBytes(x->data_type(), rows, cols);
    CheckOk(ofq_fused_layer_norm_min_max_observer(
                RawStream(ctx), x->dptr(), gamma ? gamma->dptr() : nullptr,
                beta ? beta->dptr() : nullptr, y, scale->mut_dptr<float>(),
                zero_point->mut_dptr<float>(), dt, rows, cols, epsilon, bits, y + y_bytes,
                tmp_bytes - y_bytes),
            "fused_layer_norm_min_max_observer");
    CheckOk(ofq_quantization(RawStream(ctx), y, scale->dptr(), zero_point->dptr(), out->mut_dptr(),
                             dt, OFQ_I8, rows * cols, 1, bits, OFQ_SCHEME_SYMMETRIC,
                             OFQ_FORMULA_GOOGLE, OFQ_ZP_FLOAT),
            "quantization");
  }
  bool AlwaysComputeWhenAllOutputsEmpty() const override { return false; }
};

#define REGISTER_OFQ_LN_QUANTIZATION(dtype)                                                    \
  REGISTER_USER_KERNEL("fused_layer_norm_quantization")                                        \
      .SetCreateFn<OfqLayerNormQuantizationKernel>()                                           \
      .SetIsMatchedHob((user_op::HobDeviceType() == DeviceType::kCUDA)                         \
                       && (user_op::HobDataType("x", 0) == dtype))                             \
      .SetInferTmpSizeFn([](user_op::InferContext* ctx) -> size_t {                            \
        const ShapeView xs = ctx->InputShape("x", 0);                                          \
        const int64_t cols = xs.At(xs.NumAxes() - 1);                                          \
        return LnQuantTmpBytes(dtype, xs.elem_cnt() / cols, cols);                             \
      })                                                                                       \
      .SetPriority(user_op::kKernelPriorityOptimized)
REGISTER_OFQ_LN_QUANTIZATION(DataType::kFloat16);
REGISTER_OFQ_LN_QUANTIZATION(DataType::kBFloat16);
REGISTER_OFQ_LN_QUANTIZATION(DataType::kFloat);

// ---- matmul_quant: a [m,k] int8, b [n,k] int8, a_scale [1] float, b_scale [n] float, [bias]
//      -> out [m,n] (operand layout of fused_matmul_bias, OneFlowUserOps.td:5615-5633) ----------
class OfqMatmulQuantKernel final : public user_op::OpKernel, public user_op::CudaGraphSupport {
 public:
  using user_op::OpKernel::Compute;
  void Compute(user_op::KernelComputeContext* ctx, user_op::OpKernelState*,
               const user_op::OpKernelCache*) const override {
    const user_op::Tensor* a = ctx->Tensor4ArgNameAndIndex("a", 0);
    const user_op::Tensor* b = ctx->Tensor4ArgNameAndIndex("b", 0);
    const user_op::Tensor* a_scale = ctx->Tensor4ArgNameAndIndex("a_scale", 0);
    const user_op::Tensor* b_scale = ctx->Tensor4ArgNameAndIndex("b_scale", 0);
    const user_op::Tensor* bias =
        ctx->has_input("bias", 0) ? ctx->Tensor4ArgNameAndIndex("bias", 0) : nullptr;
    user_op::Tensor* out = ctx->Tensor4ArgNameAndIndex("out", 0);
    CHECK_EQ(a->data_type(), DataType::kInt8);
    CHECK_EQ(b->data_type(), DataType::kInt8);
    CHECK_EQ(a_scale->data_type(), DataType::kFloat);
    CHECK_EQ(b_scale->data_type(), DataType::kFloat);
    CHECK_GE(a->shape_view().NumAxes(), 2);
    CHECK_EQ(b->shape_view().NumAxes(), 2);
    const int64_t k = a->shape_view().At(a->shape_view().NumAxes() - 1);
    const int64_t m = a->shape_view().elem_cnt() / k;
    const int64_t n = b->shape_view().At(0);
    CHECK_EQ(b->shape_view().At(1), k);
    CHECK_EQ(a_scale->shape_view().elem_cnt(), 1);
    CHECK_EQ(b_scale->shape_view().elem_cnt(), n);
    if (bias != nullptr) {
      CHECK_EQ(bias->shape_view().elem_cnt(), n);
      CHECK_EQ(bias->data_type(), out->data_type());
    }
    user_op::Tensor* tmp = ctx->Tensor4ArgNameAndIndex("tmp_buffer", 0);
    CheckOk(ofq_matmul_quant_ws(RawStream(ctx), a->dptr(), b->dptr(), a_scale->dptr<float>(),
                                b_scale->dptr<float>(), bias ? bias->dptr() : nullptr,
                                out->mut_dptr(), ToOfq(out->data_type()), m, n, k,
                                tmp ? tmp->mut_dptr() : nullptr,
                                tmp ? (size_t)tmp->shape_view().elem_cnt() : 0),
            "matmul_quant");
  }
  bool AlwaysComputeWhenAllOutputsEmpty() const override { return false; }
};

#define REGISTER_OFQ_MATMUL_QUANT(dtype)                                    \
  REGISTER_USER_KERNEL("matmul_quant")                                      \
      .SetCreateFn<OfqMatmulQuantKernel>()                                  \
      .SetIsMatchedHob((user_op::HobDeviceType() == DeviceType::kCUDA)      \
                       && (user_op::HobDataType("out", 0) == dtype))        \
      .SetInferTmpSizeFn([](user_op::InferContext* ctx) -> size_t {         \
        const ShapeView as = ctx->InputShape("a", 0);                       \
        const int64_t k = as.At(as.NumAxes() - 1);                          \
        return ofq_matmul_quant_workspace_bytes(as.elem_cnt() / k,          \
                                                ctx->InputShape("b", 0).At(0), k); \
      })                                                                    \
      .SetPriority(user_op::kKernelPriorityOptimized)
REGISTER_OFQ_MATMUL_QUANT(DataType::kFloat16);
REGISTER_OFQ_MATMUL_QUANT(DataType::kBFloat16);
REGISTER_OFQ_MATMUL_QUANT(DataType::kFloat);

// ---- fused_glu_with_groupwise_quantized_weight: the arguments of fused_glu
//      (x, w, [b], [v], [c] -> y, matmul_wx, [matmul_vx]; attr activation,
//      fused_glu_kernel.cu:566-600) plus w_scale, [w_zero], [v_scale], [v_zero] and the
//      quantisation attrs of the fused linear ----------------------------------------------------
class OfqFusedGluKernel final : public user_op::OpKernel, public user_op::CudaGraphSupport {
 public:
  using user_op::OpKernel::Compute;
  void Compute(user_op::KernelComputeContext* ctx, user_op::OpKernelState*,
               const user_op::OpKernelCache*) const override {
    auto opt = [&](const char* name) -> const user_op::Tensor* {
      return ctx->has_input(name, 0) ? ctx->Tensor4ArgNameAndIndex(name, 0) : nullptr;
    };
    auto ptr = [](const user_op::Tensor* t) -> const void* { return t ? t->dptr() : nullptr; };
    const user_op::Tensor* x = ctx->Tensor4ArgNameAndIndex("x", 0);
    const user_op::Tensor* w = ctx->Tensor4ArgNameAndIndex("w", 0);
    const user_op::Tensor* w_scale = ctx->Tensor4ArgNameAndIndex("w_scale", 0);
    const user_op::Tensor* v = opt("v");
    user_op::Tensor* y = ctx->Tensor4ArgNameAndIndex("y", 0);
    user_op::Tensor* matmul_wx = ctx->Tensor4ArgNameAndIndex("matmul_wx", 0);
    user_op::Tensor* matmul_vx = ctx->Tensor4ArgNameAndIndex("matmul_vx", 0);
    const std::string act = ctx->Attr<std::string>("activation");
    int act_code = -1;
    const char* names[] = {"none", "sigmoid", "relu", "gelu", "fast_gelu", "silu"};
    for (int i = 0; i < 6; ++i) {
      if (act == names[i]) act_code = i;
    }
    CHECK_GE(act_code, 0);
    const int32_t num_bits = ctx->Attr<int32_t>("num_bits");
    CHECK_GE(x->shape_view().NumAxes(), 2);
    const int64_t k = x->shape_view().At(x->shape_view().NumAxes() - 1);
    const int64_t m = x->shape_view().elem_cnt() / k;
    CHECK_EQ(w->shape_view().NumAxes(), 2);
    CHECK_EQ(w->shape_view().At(1) * (8 / num_bits), k);
    const int64_t n = v != nullptr ? w->shape_view().At(0) : w->shape_view().At(0) / 2;
    if (v != nullptr) {
      CHECK(v->shape_view() == w->shape_view());
      CHECK(matmul_vx != nullptr);
    }
    CHECK_EQ(y->shape_view().At(y->shape_view().NumAxes() - 1), n);
    CheckOk(ofq_fused_glu_gq(RawStream(ctx), x->dptr(), w->dptr(), w_scale->dptr(),
                             ptr(opt("w_zero")), ptr(opt("b")), ptr(v), ptr(opt("v_scale")),
                             ptr(opt("v_zero")), ptr(opt("c")), y->mut_dptr(),
                             matmul_wx->mut_dptr(), matmul_vx ? matmul_vx->mut_dptr() : nullptr,
                             act_code, ToOfq(w->data_type()), ToOfq(x->data_type()), num_bits,
                             ctx->Attr<bool>("symmetric") ? 1 : 0,
                             (int)ctx->Attr<int64_t>("group_dim"),
                             ctx->Attr<int64_t>("group_size"), m, n, k),
            "fused_glu_with_groupwise_quantized_weight");
  }
  bool AlwaysComputeWhenAllOutputsEmpty() const override { return false; }
};

#define REGISTER_OFQ_FUSED_GLU(dtype)                                       \
  REGISTER_USER_KERNEL("fused_glu_with_groupwise_quantized_weight")         \
      .SetCreateFn<OfqFusedGluKernel>()                                     \
      .SetIsMatchedHob((user_op::HobDeviceType() == DeviceType::kCUDA)      \
                       && (user_op::HobDataType("y", 0) == dtype))          \
      .SetPriority(user_op::kKernelPriorityOptimized)
REGISTER_OFQ_FUSED_GLU(DataType::kFloat16);
REGISTER_OFQ_FUSED_GLU(DataType::kBFloat16);
REGISTER_OFQ_FUSED_GLU(DataType::kFloat);

// ---- grouped_linear_with_groupwise_quantized_weight: variadic xs, ws, w_scales, [w_zeros],
//      [bs] -> ys, walked like GroupedMatmulBiasKernel::Compute walks its tuples
//      (grouped_matmul_bias.cu:153-190) ----------------------------------------------------------
class OfqGroupedLinearKernel final : public user_op::OpKernel, public user_op::CudaGraphSupport {
 public:
  using user_op::OpKernel::Compute;
  void Compute(user_op::KernelComputeContext* ctx, user_op::OpKernelState*,
               const user_op::OpKernelCache*) const override {
    const int32_t count = ctx->input_size("xs");
    CHECK_GE(count, 1);
    CHECK_LE(count, 64);
    CHECK_EQ(ctx->input_size("ws"), count);
    CHECK_EQ(ctx->input_size("w_scales"), count);
    const bool has_zeros = ctx->has_input("w_zeros", 0);
    const bool has_biases = ctx->has_input("bs", 0);
    if (has_zeros) { CHECK_EQ(ctx->input_size("w_zeros"), count); }
    if (has_biases) { CHECK_EQ(ctx->input_size("bs"), count); }
    const int32_t num_bits = ctx->Attr<int32_t>("num_bits");
    const void* xs[64];
    const void* ws[64];
    const void* scales[64];
    const void* zeros[64];
    const void* bs[64];
    void* ys[64];
    int64_t ms[64], ns[64], ks[64];
    for (int32_t i = 0; i < count; ++i) {
      const user_op::Tensor* x = ctx->Tensor4ArgNameAndIndex("xs", i);
      const user_op::Tensor* w = ctx->Tensor4ArgNameAndIndex("ws", i);
      CHECK_GE(x->shape_view().NumAxes(), 2);
      ks[i] = x->shape_view().At(x->shape_view().NumAxes() - 1);
      ms[i] = x->shape_view().elem_cnt() / ks[i];
      CHECK_EQ(w->shape_view().NumAxes(), 2);
      CHECK_EQ(w->shape_view().At(1) * (8 / num_bits), ks[i]);
      ns[i] = w->shape_view().At(0);
      xs[i] = x->dptr();
      ws[i] = w->dptr();
      scales[i] = ctx->Tensor4ArgNameAndIndex("w_scales", i)->dptr();
      zeros[i] = has_zeros ? ctx->Tensor4ArgNameAndIndex("w_zeros", i)->dptr() : nullptr;
      bs[i] = has_biases ? ctx->Tensor4ArgNameAndIndex("bs", i)->dptr() : nullptr;
      ys[i] = ctx->Tensor4ArgNameAndIndex("ys", i)->mut_dptr();
    }
    const user_op::Tensor* x0 = ctx->Tensor4ArgNameAndIndex("xs", 0);
    const user_op::Tensor* w0 = ctx->Tensor4ArgNameAndIndex("ws", 0);
    CheckOk(ofq_grouped_linear_gq(RawStream(ctx), count, xs, ws, scales,
                                  has_zeros ? zeros : nullptr, has_biases ? bs : nullptr, ys, ms,
                                  ns, ks, ToOfq(w0->data_type()), ToOfq(x0->data_type()), num_bits,
                                  ctx->Attr<bool>("symmetric") ? 1 : 0,
                                  (int)ctx->Attr<int64_t>("group_dim"),
                                  ctx->Attr<int64_t>("group_size")),
            "grouped_linear_with_groupwise_quantized_weight");
  }
  bool AlwaysComputeWhenAllOutputsEmpty() const override { return false; }
};

#define REGISTER_OFQ_GROUPED_LINEAR(dtype)                                  \
  REGISTER_USER_KERNEL("grouped_linear_with_groupwise_quantized_weight")    \
      .SetCreateFn<OfqGroupedLinearKernel>()                                \
      .SetIsMatchedHob((user_op::HobDeviceType() == DeviceType::kCUDA)      \
                       && (user_op::HobDataType("ys", 0) == dtype))         \
      .SetPriority(user_op::kKernelPriorityOptimized)
REGISTER_OFQ_GROUPED_LINEAR(DataType::kFloat16);
REGISTER_OFQ_GROUPED_LINEAR(DataType::kBFloat16);
REGISTER_OFQ_GROUPED_LINEAR(DataType::kFloat);

}  // namespace oneflow

#ifdef OFQ_PLUGIN_STANDALONE
// ---- test hooks of the standalone build ---------------------------------------------------------
using namespace oneflow;

namespace {
const user_op::KernelRegistration* Lookup(const std::string& op, const user_op::KernelRegContext& c) {
  const user_op::KernelRegistration* best = nullptr;
  for (const auto& r : user_op::KernelRegistry()) {
    if (r.op_type_name == op && r.matched(c) && (best == nullptr || r.priority > best->priority)) {
      best = &r;
    }
  }
  return best;
}

int CurrentDevice() {
  int dev = 0;
  if (ofq_hip_get_device(&dev) != 0) dev = 0;
  return dev;
}

// the message of the last failed GetAsyncError of a hook, for ofq_plugin_last_async_error
thread_local std::string g_last_async_error;

// What the runtime does around a kernel (stateful_opkernel.cpp:1006-1007): Compute, then ask the
// stream for an asynchronous error.  The runtime aborts on one (CHECK_JUST); the hooks return -2
// and keep the message so that a test can look at it.
int ComputeLikeTheRuntime(const user_op::OpKernel& kernel, user_op::KernelComputeContext* ctx) {
  kernel.Compute(ctx, nullptr, nullptr);
  const Maybe<void> err = ctx->stream()->GetAsyncError();
  if (err.IsOk()) return 0;
  g_last_async_error = err.error_message();
  return -2;
}

int CopyOut(const std::string& text, char* msg, int cap) {
  if (msg != nullptr && cap > 0) {
    int j = 0;
    for (; j < (int)text.size() && j < cap - 1; ++j) msg[j] = text[j];
    msg[j] = 0;
  }
  return (int)text.size();
}
}  // namespace

extern "C" int ofq_plugin_last_async_error(char* msg, int cap) {
  return CopyOut(g_last_async_error, msg, cap);
}

// ---- ep::CudaStream / ep::CudaEvent through C hooks ---------------------------------------------
extern "C" void* ofq_plugin_stream_new(int device) { return new ep::CudaStream(device); }
extern "C" void* ofq_plugin_stream_view(int device, void* raw) {
  return new ep::CudaStream(device, raw);
}
extern "C" void ofq_plugin_stream_delete(void* s) { delete static_cast<ep::CudaStream*>(s); }
extern "C" void* ofq_plugin_stream_raw(void* s) {
  // the way a kernel reaches it: through the base class and As<>
  ep::Stream* base = static_cast<ep::CudaStream*>(s);
  return base->As<ep::CudaStream>()->cuda_stream();
}
extern "C" int ofq_plugin_stream_device_type(void* s) {
  return (int)static_cast<ep::Stream*>(static_cast<ep::CudaStream*>(s))->device_type();
}
extern "C" int ofq_plugin_stream_sync(void* s, char* msg, int cap) {
  const Maybe<void> r = static_cast<ep::Stream*>(static_cast<ep::CudaStream*>(s))->Sync();
  if (r.IsOk()) return 0;
  CopyOut(r.error_message(), msg, cap);
  return -1;
}
extern "C" int ofq_plugin_stream_get_async_error(void* s, char* msg, int cap) {
  const Maybe<void> r = static_cast<ep::Stream*>(static_cast<ep::CudaStream*>(s))->GetAsyncError();
  if (r.IsOk()) return 0;
  CopyOut(r.error_message(), msg, cap);
  return -1;
}
extern "C" int ofq_plugin_stream_on_execution_context_setup(void* s) {
  ep::Stream* base = static_cast<ep::CudaStream*>(s);
  return base->OnExecutionContextSetup().IsOk() && base->OnExecutionContextTeardown().IsOk() ? 0 : -1;
}
extern "C" int ofq_plugin_stream_cu_count(void* s) {
  return static_cast<ep::CudaStream*>(s)->multi_processor_count();
}
extern "C" unsigned ofq_plugin_stream_grid_with_waves(void* s, size_t elem_cnt, size_t block_size,
                                                      size_t max_waves) {
  ep::CudaLaunchConfig config;
  static_cast<ep::CudaStream*>(s)->InitLaunchConfigWithWaves(&config, elem_cnt, block_size, max_waves);
  return config.grid_dim;
}
extern "C" void* ofq_plugin_event_new() { return new ep::CudaEvent(0); }
extern "C" void ofq_plugin_event_delete(void* e) { delete static_cast<ep::CudaEvent*>(e); }
extern "C" void ofq_plugin_stream_record_event(void* s, void* e) {
  static_cast<ep::Stream*>(static_cast<ep::CudaStream*>(s))->RecordEvent(static_cast<ep::CudaEvent*>(e));
}
extern "C" void ofq_plugin_stream_wait_event(void* s, void* e) {
  static_cast<ep::Stream*>(static_cast<ep::CudaStream*>(s))->WaitEvent(static_cast<ep::CudaEvent*>(e));
}
// 1 done, 0 pending, -1 error
extern "C" int ofq_plugin_event_query_done(void* e) {
  const Maybe<bool> r = static_cast<ep::Event*>(static_cast<ep::CudaEvent*>(e))->QueryDone();
  return r.IsOk() ? (r.value() ? 1 : 0) : -1;
}
extern "C" int ofq_plugin_event_sync(void* e) {
  return static_cast<ep::Event*>(static_cast<ep::CudaEvent*>(e))->Sync().IsOk() ? 0 : -1;
}

extern "C" int ofq_plugin_registration_count() { return (int)user_op::KernelRegistry().size(); }

extern "C" int ofq_plugin_registration_info(int i, char* name, int name_cap, int* priority,
                                            int* needs_tmp) {
  const auto& regs = user_op::KernelRegistry();
  if (i < 0 || i >= (int)regs.size()) return -1;
  const std::string& n = regs[i].op_type_name;
  int j = 0;
  for (; j < (int)n.size() && j < name_cap - 1; ++j) name[j] = n[j];
  name[j] = 0;
  *priority = regs[i].priority;
  *needs_tmp = regs[i].infer_tmp_size ? 1 : 0;
  return 0;
}

// 1 if a kernel is registered for (op, device, dtype of `arg`)
extern "C" int ofq_plugin_has_kernel(const char* op, int device, const char* arg, int dtype) {
  user_op::KernelRegContext c;
  c.device = (DeviceType)device;
  c.arg_dtypes[arg] = (DataType)dtype;
  return Lookup(op, c) != nullptr ? 1 : 0;
}

// tmp_buffer bytes the observer registration asks the runtime for
extern "C" long long ofq_plugin_observer_tmp_bytes(int dtype, const long long* shape, int rank,
                                                   int per_layer) {
  user_op::KernelRegContext c;
  c.device = DeviceType::kCUDA;
  c.arg_dtypes["in"] = (DataType)dtype;
  const auto* r = Lookup("min_max_observer", c);
  if (r == nullptr || !r->infer_tmp_size) return -1;
  user_op::InferContext ic;
  ic.shapes["in"] = std::vector<int64_t>(shape, shape + rank);
  ic.attrs["per_layer_quantization"].b = per_layer != 0;
  return (long long)r->infer_tmp_size(&ic);
}

// tmp_buffer size the fused linear registration asks for (2-D x)
extern "C" long long ofq_plugin_fused_linear_tmp_bytes(int t_dtype, int w_dtype, long long m,
                                                       long long n, long long k, int num_bits,
                                                       int symmetric, long long group_dim,
                                                       long long group_size) {
  user_op::KernelRegContext c;
  c.device = DeviceType::kCUDA;
  c.arg_dtypes["out"] = (DataType)t_dtype;
  const auto* r = Lookup("fused_linear_with_groupwise_quantized_weight", c);
  if (r == nullptr || !r->infer_tmp_size) return -1;
  user_op::InferContext ic;
  ic.shapes["x"] = {m, k};
  ic.shapes["w"] = {n, k * num_bits / 8};
  ic.dtypes["w"] = (DataType)w_dtype;
  ic.attrs["num_bits"].i = num_bits;
  ic.attrs["symmetric"].b = symmetric != 0;
  ic.attrs["group_dim"].i = group_dim;
  ic.attrs["group_size"].i = group_size;
  return (long long)r->infer_tmp_size(&ic);
}

// Runs the registered fused linear kernel on device pointers through a KernelComputeContext,
// the way the runtime would (2-D x).
extern "C" int ofq_plugin_run_fused_linear(void* stream, void* x, void* w, void* w_scale,
                                           void* w_zero, void* b, void* out, int t_dtype,
                                           int w_dtype, long long m, long long n, long long k,
                                           int num_bits, int symmetric, long long group_dim,
                                           long long group_size) {
  user_op::KernelRegContext c;
  c.device = DeviceType::kCUDA;
  c.arg_dtypes["out"] = (DataType)t_dtype;
  const auto* r = Lookup("fused_linear_with_groupwise_quantized_weight", c);
  if (r == nullptr) return -1;
  ep::CudaStream st(CurrentDevice(), stream);
  user_op::KernelComputeContext ctx;
  ctx.stream_ = &st;
  const DataType T = (DataType)t_dtype;
  const int64_t groups = (group_dim == 0 ? n : k) / group_size;
  ctx.AddTensor("x", {m, k}, T, x);
  ctx.AddTensor("w", {n, k * num_bits / 8}, (DataType)w_dtype, w);
  if (group_dim == 0) {
    ctx.AddTensor("w_scale", {groups, k}, T, w_scale);
    if (w_zero) ctx.AddTensor("w_zero", {groups, k}, T, w_zero);
  } else {
    ctx.AddTensor("w_scale", {n, groups}, T, w_scale);
    if (w_zero) ctx.AddTensor("w_zero", {n, groups}, T, w_zero);
  }
  if (b) ctx.AddTensor("b", {n}, T, b);
  ctx.AddTensor("out", {m, n}, T, out);
  ctx.attrs["num_bits"].i = num_bits;
  ctx.attrs["symmetric"].b = symmetric != 0;
  ctx.attrs["group_dim"].i = group_dim;
  ctx.attrs["group_size"].i = group_size;
  auto kernel = r->create();
  return ComputeLikeTheRuntime(*kernel, &ctx);
}
// Runs the registered dynamic-int8 front end (LayerNorm + observer, with the optional residual
// inputs) through a KernelComputeContext.
extern "C" int ofq_plugin_run_layer_norm_observer(void* stream, void* x, void* gamma, void* beta,
                                                  void* bias, void* skip, double alpha, void* y,
                                                  void* scale, void* zero_point, void* tmp,
                                                  long long tmp_bytes, int t_dtype, long long rows,
                                                  long long cols, double epsilon, int bits) {
  user_op::KernelRegContext c;
  c.device = DeviceType::kCUDA;
  c.arg_dtypes["y"] = (DataType)t_dtype;
  const auto* r = Lookup("fused_layer_norm_min_max_observer", c);
  if (r == nullptr) return -1;
  ep::CudaStream st(CurrentDevice(), stream);
  user_op::KernelComputeContext ctx;
  ctx.stream_ = &st;
  const DataType T = (DataType)t_dtype;
  ctx.AddTensor("x", {rows, cols}, T, x);
  if (gamma) ctx.AddTensor("gamma", {cols}, T, gamma);
  if (beta) ctx.AddTensor("beta", {cols}, T, beta);
  if (bias) ctx.AddTensor("bias", {cols}, T, bias);
  if (skip) ctx.AddTensor("skip", {rows, cols}, T, skip);
  ctx.AddTensor("y", {rows, cols}, T, y);
  ctx.AddTensor("scale", {1}, DataType::kFloat, scale);
  ctx.AddTensor("zero_point", {1}, DataType::kFloat, zero_point);
  ctx.AddTensor("tmp_buffer", {tmp_bytes}, DataType::kUInt8, tmp);
  ctx.attrs["epsilon"].f = epsilon;
  ctx.attrs["alpha"].f = alpha;
  ctx.attrs["quantization_bit"].i = bits;
  auto kernel = r->create();
  return ComputeLikeTheRuntime(*kernel, &ctx);
}

// Runs the registered LayerNorm -> int8 kernel; tmp must hold ofq_plugin_ln_quantization_tmp_bytes.
extern "C" long long ofq_plugin_ln_quantization_tmp_bytes(int t_dtype, long long rows,
                                                          long long cols) {
  user_op::KernelRegContext c;
  c.device = DeviceType::kCUDA;
  c.arg_dtypes["x"] = (DataType)t_dtype;
  const auto* r = Lookup("fused_layer_norm_quantization", c);
  if (r == nullptr || !r->infer_tmp_size) return -1;
  user_op::InferContext ic;
  ic.shapes["x"] = {rows, cols};
  return (long long)r->infer_tmp_size(&ic);
}
extern "C" int ofq_plugin_run_layer_norm_quantization(void* stream, void* x, void* gamma,
                                                      void* beta, void* out, void* scale,
                                                      void* zero_point, void* tmp,
                                                      long long tmp_bytes, int t_dtype,
                                                      long long rows, long long cols,
                                                      double epsilon, int bits) {
  user_op::KernelRegContext c;
  c.device = DeviceType::kCUDA;
  c.arg_dtypes["x"] = (DataType)t_dtype;
  const auto* r = Lookup("fused_layer_norm_quantization", c);
  if (r == nullptr) return -1;
  ep::CudaStream st(CurrentDevice(), stream);
  user_op::KernelComputeContext ctx;
  ctx.stream_ = &st;
  const DataType T = (DataType)t_dtype;
  ctx.AddTensor("x", {rows, cols}, T, x);
  if (gamma) ctx.AddTensor("gamma", {cols}, T, gamma);
  if (beta) ctx.AddTensor("beta", {cols}, T, beta);
  ctx.AddTensor("out", {rows, cols}, DataType::kInt8, out);
  ctx.AddTensor("scale", {1}, DataType::kFloat, scale);
  ctx.AddTensor("zero_point", {1}, DataType::kFloat, zero_point);
  ctx.AddTensor("tmp_buffer", {tmp_bytes}, DataType::kUInt8, tmp);
  ctx.attrs["epsilon"].f = epsilon;
  ctx.attrs["quantization_bit"].i = bits;
  auto kernel = r->create();
  return ComputeLikeTheRuntime(*kernel, &ctx);
}

extern "C" int ofq_plugin_run_matmul_quant(void* stream, void* a, void* b, void* a_scale,
                                           void* b_scale, void* bias, void* out, int out_dtype,
                                           long long m, long long n, long long k) {
  user_op::KernelRegContext c;
  c.device = DeviceType::kCUDA;
  c.arg_dtypes["out"] = (DataType)out_dtype;
  const auto* r = Lookup("matmul_quant", c);
  if (r == nullptr) return -1;
  ep::CudaStream st(CurrentDevice(), stream);
  user_op::KernelComputeContext ctx;
  ctx.stream_ = &st;
  ctx.AddTensor("a", {m, k}, DataType::kInt8, a);
  ctx.AddTensor("b", {n, k}, DataType::kInt8, b);
  ctx.AddTensor("a_scale", {1}, DataType::kFloat, a_scale);
  ctx.AddTensor("b_scale", {n}, DataType::kFloat, b_scale);
  if (bias) ctx.AddTensor("bias", {n}, (DataType)out_dtype, bias);
  ctx.AddTensor("out", {m, n}, (DataType)out_dtype, out);
  auto kernel = r->create();
  return ComputeLikeTheRuntime(*kernel, &ctx);
}

// q/k/v-style grouped call: `count` problems sharing x ([m,k]) with weights [ns[i], k*bits/8]
// (symmetric, groups along K), outputs ys[i] [m, ns[i]]
extern "C" int ofq_plugin_run_grouped_linear(void* stream, int count, void* x, void** ws,
                                             void** scales, void** ys, const long long* ns,
                                             int t_dtype, int w_dtype, long long m, long long k,
                                             int num_bits, long long group_size) {
  user_op::KernelRegContext c;
  c.device = DeviceType::kCUDA;
  c.arg_dtypes["ys"] = (DataType)t_dtype;
  const auto* r = Lookup("grouped_linear_with_groupwise_quantized_weight", c);
  if (r == nullptr) return -1;
  ep::CudaStream st(CurrentDevice(), stream);
  user_op::KernelComputeContext ctx;
  ctx.stream_ = &st;
  const DataType T = (DataType)t_dtype;
  for (int i = 0; i < count; ++i) {
    ctx.AddTensor("xs", {m, k}, T, x, i);
    ctx.AddTensor("ws", {ns[i], k * num_bits / 8}, (DataType)w_dtype, ws[i], i);
    ctx.AddTensor("w_scales", {ns[i], k / group_size}, T, scales[i], i);
    ctx.AddTensor("ys", {m, ns[i]}, T, ys[i], i);
  }
  ctx.attrs["num_bits"].i = num_bits;
  ctx.attrs["symmetric"].b = true;
  ctx.attrs["group_dim"].i = 1;
  ctx.attrs["group_size"].i = group_size;
  auto kernel = r->create();
  return ComputeLikeTheRuntime(*kernel, &ctx);
}
#endif  // OFQ_PLUGIN_STANDALONE
