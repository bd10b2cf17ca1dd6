// Op definitions (shape and dtype inference) of the four ops this library adds next to the
// reference's quantization ops.  The reference pairs every kernel with such a definition:
//   oneflow/user/ops/fused_linear_with_groupwise_quantized_weight_op.cpp:27-94 (tensor descs and
//   dtypes of the fused linear), oneflow/user/ops/fused_glu_op.cpp (fused_glu),
//   oneflow/user/ops/grouped_matmul_bias_op.cpp (grouped_matmul_bias),
//   oneflow/user/ops/skip_layer_norm_op.cpp, min_max_observer_op.cpp (the two halves of the fused
//   LayerNorm + observer), schema in oneflow/ir/include/OneFlow/OneFlowUserOps.td:8248-8387.
// The functions below are what the generated op classes' static InferLogicalTensorDesc /
// InferPhysicalTensorDesc / InferDataType would forward to (same signatures, same CHECK_*_OR_RETURN
// style, same argument names as the kernels in ofq_oneflow_kernels.cpp).  SBP signatures
// (GetSbp) are left out: nothing here runs on more than one device; the signatures the ops would
// carry are those of fused_linear_with_groupwise_quantized_weight_op.cpp:125-177 (split n with x
// broadcast, split k with partial sums) for the linears and split over rows for the LayerNorm.
#include "oneflow/core/framework/framework.h"

namespace oneflow {

namespace {

// the weight / scale / zero rules of one groupwise-quantised linear [n, k]: returns n
Maybe<void> CheckQuantizedWeight(user_op::InferContext* ctx, const std::string& w_name,
                                 const std::string& scale_name, const std::string& zero_name,
                                 int32_t index, int64_t k, int64_t* n_out) {
  const user_op::TensorDesc& w_desc = ctx->InputTensorDesc(w_name, index);
  CHECK_EQ_OR_RETURN(w_desc.shape().NumAxes(), 2);
  const int64_t n = w_desc.shape().At(0);
  const int32_t num_bits = ctx->Attr<int32_t>("num_bits");
  if (num_bits == 8) {
    CHECK_EQ_OR_RETURN(w_desc.shape().At(1), k);
  } else if (num_bits == 4) {
    CHECK_EQ_OR_RETURN(w_desc.shape().At(1) * 2, k);
  } else {
    UNIMPLEMENTED_THEN_RETURN();
  }
  const int64_t group_dim = ctx->Attr<int64_t>("group_dim");
  CHECK_OR_RETURN(group_dim == 0 || group_dim == 1);
  const int64_t group_dim_size = group_dim == 0 ? n : k;
  const int64_t group_size = ctx->Attr<int64_t>("group_size");
  CHECK_GT_OR_RETURN(group_size, 1);
  CHECK_LE_OR_RETURN(group_size, group_dim_size);
  CHECK_EQ_OR_RETURN(group_dim_size % group_size, 0);
  const int64_t num_groups = group_dim_size / group_size;
  const user_op::TensorDesc& scale_desc = ctx->InputTensorDesc(scale_name, index);
  CHECK_EQ_OR_RETURN(scale_desc.shape().NumAxes(), 2);
  if (group_dim == 0) {
    CHECK_EQ_OR_RETURN(scale_desc.shape().At(0), num_groups);
    CHECK_EQ_OR_RETURN(scale_desc.shape().At(1), k);
  } else {
    CHECK_EQ_OR_RETURN(scale_desc.shape().At(0), n);
    CHECK_EQ_OR_RETURN(scale_desc.shape().At(1), num_groups);
  }
  if (ctx->has_input(zero_name, index)) {
    CHECK_OR_RETURN(ctx->InputTensorDesc(zero_name, index).shape() == scale_desc.shape());
  }
  *n_out = n;
  return Maybe<void>::Ok();
}

Maybe<void> CheckQuantizedDtypes(user_op::InferContext* ctx, DataType data_type,
                                 const std::string& w_name, const std::string& scale_name,
                                 const std::string& zero_name, const std::string& bias_name,
                                 int32_t index) {
  CHECK_EQ_OR_RETURN(ctx->InputDType(scale_name, index), data_type);
  if (ctx->has_input(zero_name, index)) {
    CHECK_EQ_OR_RETURN(ctx->InputDType(zero_name, index), data_type);
  }
  if (ctx->has_input(bias_name, index)) {
    CHECK_EQ_OR_RETURN(ctx->InputDType(bias_name, index), data_type);
  }
  if (ctx->Attr<bool>("symmetric")) {
    CHECK_OR_RETURN(ctx->InputDType(w_name, index) == DataType::kUInt8
                    || ctx->InputDType(w_name, index) == DataType::kInt8);
    CHECK_OR_RETURN(!ctx->has_input(zero_name, index));
  } else {
    CHECK_EQ_OR_RETURN(ctx->InputDType(w_name, index), DataType::kUInt8);
    CHECK_OR_RETURN(ctx->has_input(zero_name, index));
  }
  return Maybe<void>::Ok();
}

}  // namespace

// ---- fused_layer_norm_min_max_observer: x, [gamma], [beta], [bias], [skip] -> y, scale,
//      zero_point; attrs epsilon, alpha (double), quantization_bit (int32) ------------------------
struct FusedLayerNormMinMaxObserverOp {
  static Maybe<void> InferLogicalTensorDesc(user_op::InferContext* ctx) {
    const user_op::TensorDesc& x_desc = ctx->InputTensorDesc("x", 0);
    // (skip_layer_norm_op.cpp: x has at least two axes, the parameters are vectors over the last)
    CHECK_GE_OR_RETURN(x_desc.shape().NumAxes(), 2);
    const int64_t cols = x_desc.shape().At(x_desc.shape().NumAxes() - 1);
    for (const char* name : {"gamma", "beta", "bias"}) {
      if (ctx->has_input(name, 0)) {
        const user_op::TensorDesc& d = ctx->InputTensorDesc(name, 0);
        CHECK_EQ_OR_RETURN(d.shape().NumAxes(), 1);
        CHECK_EQ_OR_RETURN(d.shape().At(0), cols);
      }
    }
    if (ctx->has_input("skip", 0)) {
      CHECK_OR_RETURN(ctx->InputTensorDesc("skip", 0).shape() == x_desc.shape());
    }
    // (min_max_observer_op.cpp:47-54: the attribute domain; per-layer: one scale, one zero point)
    const int32_t quantization_bit = ctx->Attr<int32_t>("quantization_bit");
    CHECK_GT_OR_RETURN(quantization_bit, 1);
    CHECK_LE_OR_RETURN(quantization_bit, 8);
    CHECK_GE_OR_RETURN(ctx->Attr<double>("epsilon"), 0.0);
    ctx->SetOutputShape("y", 0, x_desc.shape());
    ctx->SetOutputShape("scale", 0, Shape({1}));
    ctx->SetOutputShape("zero_point", 0, Shape({1}));
    return Maybe<void>::Ok();
  }
  static Maybe<void> InferPhysicalTensorDesc(user_op::InferContext* ctx) {
    return InferLogicalTensorDesc(ctx);
  }
  static Maybe<void> InferDataType(user_op::InferContext* ctx) {
    const DataType data_type = ctx->InputDType("x", 0);
    CHECK_OR_RETURN(data_type == DataType::kFloat16 || data_type == DataType::kBFloat16
                    || data_type == DataType::kFloat);
    for (const char* name : {"gamma", "beta", "bias", "skip"}) {
      if (ctx->has_input(name, 0)) { CHECK_EQ_OR_RETURN(ctx->InputDType(name, 0), data_type); }
    }
    ctx->SetOutputDType("y", 0, data_type);
    ctx->SetOutputDType("scale", 0, DataType::kFloat);
    ctx->SetOutputDType("zero_point", 0, DataType::kFloat);
    return Maybe<void>::Ok();
  }
};

// ---- fused_layer_norm_quantization: x, [gamma], [beta] -> out (int8 codes, the shape of x),
//      scale, zero_point; attrs epsilon (double), quantization_bit (int32).  The op above followed
//      by `quantization` (symmetric, per layer) of its y (quantization_op.cpp: the output has the
//      shape of the input) ------------------------------------------------------------------------
struct FusedLayerNormQuantizationOp {
  static Maybe<void> InferLogicalTensorDesc(user_op::InferContext* ctx) {
    const user_op::TensorDesc& x_desc = ctx->InputTensorDesc("x", 0);
    CHECK_GE_OR_RETURN(x_desc.shape().NumAxes(), 2);
    const int64_t cols = x_desc.shape().At(x_desc.shape().NumAxes() - 1);
    for (const char* name : {"gamma", "beta"}) {
      if (ctx->has_input(name, 0)) {
        const user_op::TensorDesc& d = ctx->InputTensorDesc(name, 0);
        CHECK_EQ_OR_RETURN(d.shape().NumAxes(), 1);
        CHECK_EQ_OR_RETURN(d.shape().At(0), cols);
      }
    }
    const int32_t quantization_bit = ctx->Attr<int32_t>("quantization_bit");
    CHECK_GT_OR_RETURN(quantization_bit, 1);
    CHECK_LE_OR_RETURN(quantization_bit, 8);
    CHECK_GE_OR_RETURN(ctx->Attr<double>("epsilon"), 0.0);
    ctx->SetOutputShape("out", 0, x_desc.shape());
    ctx->SetOutputShape("scale", 0, Shape({1}));
    ctx->SetOutputShape("zero_point", 0, Shape({1}));
    return Maybe<void>::Ok();
  }
  static Maybe<void> InferPhysicalTensorDesc(user_op::InferContext* ctx) {
    return InferLogicalTensorDesc(ctx);
  }
  static Maybe<void> InferDataType(user_op::InferContext* ctx) {
    const DataType data_type = ctx->InputDType("x", 0);
    CHECK_OR_RETURN(data_type == DataType::kFloat16 || data_type == DataType::kBFloat16
                    || data_type == DataType::kFloat);
    for (const char* name : {"gamma", "beta"}) {
      if (ctx->has_input(name, 0)) { CHECK_EQ_OR_RETURN(ctx->InputDType(name, 0), data_type); }
    }
    ctx->SetOutputDType("out", 0, DataType::kInt8);
    ctx->SetOutputDType("scale", 0, DataType::kFloat);
    ctx->SetOutputDType("zero_point", 0, DataType::kFloat);
    return Maybe<void>::Ok();
  }
};

// ---- matmul_quant: a [.., k] int8, b [n, k] int8, a_scale [1], b_scale [n], [bias] [n] -> out
//      [.., n]; attr out_dtype ------------------------------------------------------------------
struct MatmulQuantOp {
  static Maybe<void> InferLogicalTensorDesc(user_op::InferContext* ctx) {
    const user_op::TensorDesc& a_desc = ctx->InputTensorDesc("a", 0);
    CHECK_GE_OR_RETURN(a_desc.shape().NumAxes(), 2);
    const int64_t k = a_desc.shape().At(a_desc.shape().NumAxes() - 1);
    const user_op::TensorDesc& b_desc = ctx->InputTensorDesc("b", 0);
    CHECK_EQ_OR_RETURN(b_desc.shape().NumAxes(), 2);
    CHECK_EQ_OR_RETURN(b_desc.shape().At(1), k);
    const int64_t n = b_desc.shape().At(0);
    CHECK_EQ_OR_RETURN(ctx->InputTensorDesc("a_scale", 0).shape().elem_cnt(), 1);
    CHECK_EQ_OR_RETURN(ctx->InputTensorDesc("b_scale", 0).shape().elem_cnt(), n);
    if (ctx->has_input("bias", 0)) {
      const user_op::TensorDesc& bias_desc = ctx->InputTensorDesc("bias", 0);
      CHECK_EQ_OR_RETURN(bias_desc.shape().NumAxes(), 1);
      CHECK_EQ_OR_RETURN(bias_desc.shape().At(0), n);
    }
    Shape out_shape = a_desc.shape();
    out_shape[a_desc.shape().NumAxes() - 1] = n;
    ctx->SetOutputShape("out", 0, out_shape);
    return Maybe<void>::Ok();
  }
  static Maybe<void> InferPhysicalTensorDesc(user_op::InferContext* ctx) {
    return InferLogicalTensorDesc(ctx);
  }
  static Maybe<void> InferDataType(user_op::InferContext* ctx) {
    CHECK_EQ_OR_RETURN(ctx->InputDType("a", 0), DataType::kInt8);
    CHECK_EQ_OR_RETURN(ctx->InputDType("b", 0), DataType::kInt8);
    CHECK_EQ_OR_RETURN(ctx->InputDType("a_scale", 0), DataType::kFloat);
    CHECK_EQ_OR_RETURN(ctx->InputDType("b_scale", 0), DataType::kFloat);
    const DataType out_dtype = ctx->Attr<DataType>("out_dtype");
    CHECK_OR_RETURN(out_dtype == DataType::kFloat16 || out_dtype == DataType::kBFloat16
                    || out_dtype == DataType::kFloat);
    if (ctx->has_input("bias", 0)) { CHECK_EQ_OR_RETURN(ctx->InputDType("bias", 0), out_dtype); }
    ctx->SetOutputDType("out", 0, out_dtype);
    return Maybe<void>::Ok();
  }
};

// ---- fused_glu_with_groupwise_quantized_weight: the arguments of fused_glu (fused_glu_op.cpp:
//      x, w, [b], [v], [c] -> y, matmul_wx, [matmul_vx]) with quantised weights.  Without v the
//      one weight holds the hidden rows followed by the gate rows ([2n, k]). ------------------------
struct FusedGluWithGroupwiseQuantizedWeightOp {
  static Maybe<void> InferLogicalTensorDesc(user_op::InferContext* ctx) {
    const user_op::TensorDesc& x_desc = ctx->InputTensorDesc("x", 0);
    CHECK_GE_OR_RETURN(x_desc.shape().NumAxes(), 2);
    const int64_t k = x_desc.shape().At(x_desc.shape().NumAxes() - 1);
    int64_t w_rows = 0;
    JUST(CheckQuantizedWeight(ctx, "w", "w_scale", "w_zero", 0, k, &w_rows));
    const bool split = ctx->has_input("v", 0);
    int64_t n = w_rows;
    if (split) {
      int64_t v_rows = 0;
      JUST(CheckQuantizedWeight(ctx, "v", "v_scale", "v_zero", 0, k, &v_rows));
      CHECK_EQ_OR_RETURN(v_rows, w_rows);
      CHECK_EQ_OR_RETURN(ctx->has_input("b", 0), ctx->has_input("c", 0));
    } else {
      CHECK_OR_RETURN(!ctx->has_input("c", 0));
      CHECK_EQ_OR_RETURN(w_rows % 2, 0);
      n = w_rows / 2;
    }
    for (const char* name : {"b", "c"}) {
      if (ctx->has_input(name, 0)) {
        const user_op::TensorDesc& d = ctx->InputTensorDesc(name, 0);
        CHECK_EQ_OR_RETURN(d.shape().NumAxes(), 1);
        CHECK_EQ_OR_RETURN(d.shape().At(0), w_rows);
      }
    }
    Shape y_shape = x_desc.shape();
    y_shape[x_desc.shape().NumAxes() - 1] = n;
    Shape wx_shape = x_desc.shape();
    wx_shape[x_desc.shape().NumAxes() - 1] = w_rows;
    ctx->SetOutputShape("y", 0, y_shape);
    ctx->SetOutputShape("matmul_wx", 0, wx_shape);
    if (split) { ctx->SetOutputShape("matmul_vx", 0, y_shape); }
    return Maybe<void>::Ok();
  }
  static Maybe<void> InferPhysicalTensorDesc(user_op::InferContext* ctx) {
    return InferLogicalTensorDesc(ctx);
  }
  static Maybe<void> InferDataType(user_op::InferContext* ctx) {
    const DataType data_type = ctx->InputDType("x", 0);
    const std::string act = ctx->Attr<std::string>("activation");
    CHECK_OR_RETURN(act == "none" || act == "sigmoid" || act == "relu" || act == "gelu"
                    || act == "fast_gelu" || act == "silu");
    JUST(CheckQuantizedDtypes(ctx, data_type, "w", "w_scale", "w_zero", "b", 0));
    ctx->SetOutputDType("y", 0, data_type);
    ctx->SetOutputDType("matmul_wx", 0, data_type);
    if (ctx->has_input("v", 0)) {
      JUST(CheckQuantizedDtypes(ctx, data_type, "v", "v_scale", "v_zero", "c", 0));
      ctx->SetOutputDType("matmul_vx", 0, data_type);
    }
    return Maybe<void>::Ok();
  }
};

// ---- grouped_linear_with_groupwise_quantized_weight: variadic xs, ws, w_scales, [w_zeros], [bs]
//      -> ys (grouped_matmul_bias_op.cpp: equal counts, every problem checked on its own) ---------
struct GroupedLinearWithGroupwiseQuantizedWeightOp {
  static Maybe<void> InferLogicalTensorDesc(user_op::InferContext* ctx) {
    const int32_t count = ctx->input_size("xs");
    CHECK_GE_OR_RETURN(count, 1);
    CHECK_LE_OR_RETURN(count, 64);
    CHECK_EQ_OR_RETURN(ctx->input_size("ws"), count);
    CHECK_EQ_OR_RETURN(ctx->input_size("w_scales"), count);
    if (ctx->has_input("w_zeros", 0)) { CHECK_EQ_OR_RETURN(ctx->input_size("w_zeros"), count); }
    if (ctx->has_input("bs", 0)) { CHECK_EQ_OR_RETURN(ctx->input_size("bs"), count); }
    for (int32_t i = 0; i < count; ++i) {
      const user_op::TensorDesc& x_desc = ctx->InputTensorDesc("xs", i);
      CHECK_GE_OR_RETURN(x_desc.shape().NumAxes(), 2);
      const int64_t k = x_desc.shape().At(x_desc.shape().NumAxes() - 1);
      int64_t n = 0;
      JUST(CheckQuantizedWeight(ctx, "ws", "w_scales", "w_zeros", i, k, &n));
      if (ctx->has_input("bs", i)) {
        const user_op::TensorDesc& b_desc = ctx->InputTensorDesc("bs", i);
        CHECK_EQ_OR_RETURN(b_desc.shape().NumAxes(), 1);
        CHECK_EQ_OR_RETURN(b_desc.shape().At(0), n);
      }
      Shape out_shape = x_desc.shape();
      out_shape[x_desc.shape().NumAxes() - 1] = n;
      ctx->SetOutputShape("ys", i, out_shape);
    }
    return Maybe<void>::Ok();
  }
  static Maybe<void> InferPhysicalTensorDesc(user_op::InferContext* ctx) {
    return InferLogicalTensorDesc(ctx);
  }
  static Maybe<void> InferDataType(user_op::InferContext* ctx) {
    const int32_t count = ctx->input_size("xs");
    const DataType data_type = ctx->InputDType("xs", 0);
    for (int32_t i = 0; i < count; ++i) {
      CHECK_EQ_OR_RETURN(ctx->InputDType("xs", i), data_type);
      JUST(CheckQuantizedDtypes(ctx, data_type, "ws", "w_scales", "w_zeros", "bs", i));
      ctx->SetOutputDType("ys", i, data_type);
    }
    return Maybe<void>::Ok();
  }
};

}  // namespace oneflow

#ifdef OFQ_PLUGIN_STANDALONE
// ---- test hook: run an op definition's three inference functions on a described call ------------
// ctx: an InferContext built by ofq_plugin_infer_* calls; returns 0, or -1 with the message
using namespace oneflow;
namespace {
thread_local std::string g_infer_error;
template<class Op>
int RunInference(user_op::InferContext* ctx) {
  for (auto fn : {&Op::InferLogicalTensorDesc, &Op::InferPhysicalTensorDesc, &Op::InferDataType}) {
    const Maybe<void> r = fn(ctx);
    if (!r.IsOk()) {
      g_infer_error = r.error_message();
      return -1;
    }
  }
  return 0;
}
}  // namespace

extern "C" void* ofq_plugin_infer_new() { return new user_op::InferContext(); }
extern "C" void ofq_plugin_infer_delete(void* c) { delete static_cast<user_op::InferContext*>(c); }
extern "C" void ofq_plugin_infer_add_input(void* c, const char* name, int index,
                                           const long long* shape, int rank, int dtype) {
  static_cast<user_op::InferContext*>(c)->AddInput(
      name, index, std::vector<int64_t>(shape, shape + rank), (DataType)dtype);
}
extern "C" void ofq_plugin_infer_attr_int(void* c, const char* name, long long v) {
  static_cast<user_op::InferContext*>(c)->attrs[name].i = v;
}
extern "C" void ofq_plugin_infer_attr_bool(void* c, const char* name, int v) {
  static_cast<user_op::InferContext*>(c)->attrs[name].b = v != 0;
}
extern "C" void ofq_plugin_infer_attr_double(void* c, const char* name, double v) {
  static_cast<user_op::InferContext*>(c)->attrs[name].f = v;
}
extern "C" void ofq_plugin_infer_attr_string(void* c, const char* name, const char* v) {
  static_cast<user_op::InferContext*>(c)->attrs[name].s = v;
}
extern "C" int ofq_plugin_infer_run(void* c, const char* op) {
  auto* ctx = static_cast<user_op::InferContext*>(c);
  const std::string name = op;
  if (name == "fused_layer_norm_min_max_observer") return RunInference<FusedLayerNormMinMaxObserverOp>(ctx);
  if (name == "fused_layer_norm_quantization") return RunInference<FusedLayerNormQuantizationOp>(ctx);
  if (name == "matmul_quant") return RunInference<MatmulQuantOp>(ctx);
  if (name == "fused_glu_with_groupwise_quantized_weight") {
    return RunInference<FusedGluWithGroupwiseQuantizedWeightOp>(ctx);
  }
  if (name == "grouped_linear_with_groupwise_quantized_weight") {
    return RunInference<GroupedLinearWithGroupwiseQuantizedWeightOp>(ctx);
  }
  g_infer_error = "no such op definition: " + name;
  return -2;
}
extern "C" int ofq_plugin_infer_error(char* msg, int cap) {
  int j = 0;
  for (; j < (int)g_infer_error.size() && j < cap - 1; ++j) msg[j] = g_infer_error[j];
  if (cap > 0) msg[j] = 0;
  return (int)g_infer_error.size();
}
// rank of an output (-1: not set); its shape and dtype
extern "C" int ofq_plugin_infer_output(void* c, const char* name, int index, long long* shape,
                                       int cap, int* dtype) {
  auto* ctx = static_cast<user_op::InferContext*>(c);
  auto it = ctx->out.find({name, index});
  if (it == ctx->out.end()) return -1;
  const Shape& s = it->second.shape();
  for (int i = 0; i < s.NumAxes() && i < cap; ++i) shape[i] = s.At(i);
  *dtype = (int)it->second.data_type();
  return (int)s.NumAxes();
}
#endif  // OFQ_PLUGIN_STANDALONE
