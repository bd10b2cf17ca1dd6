// Minimal stand-alone restatement of the slice of OneFlow's user-op kernel API that the adapter
// in ofq_oneflow_kernels.cpp touches, so that the adapter can be compiled and exercised without
// a OneFlow build.  It mirrors names and call shapes of
//   oneflow/core/framework/op_kernel.h:287-324          (OpKernel, KernelComputeContext)
//   oneflow/core/framework/user_op_tensor.h:40-75        (Tensor)
//   oneflow/core/framework/user_op_kernel_registry.h:60-107, user_op_registry_manager.h:107-110
//   oneflow/core/framework/user_op_hob.h:43-73           (HobDeviceType, HobDataType)
//   oneflow/core/ep/include/stream.h:30-57               (ep::Stream)
//   oneflow/core/ep/include/event.h:26-35                (ep::Event)
//   oneflow/core/common/maybe.h, error.h                 (Maybe<void>, Maybe<bool>, Error: what
//                                                         the stream layer constructs and tests)
// When building against a real OneFlow tree this directory is simply left off the include path.
#pragma once

#include <cstdint>
#include <cstdlib>
#include <functional>
#include <iostream>
#include <map>
#include <memory>
#include <sstream>
#include <string>
#include <utility>
#include <vector>

namespace oneflow {

enum class DeviceType { kInvalidDevice = 0, kCPU = 1, kCUDA = 2 };
enum DataType {
  kInvalidDataType = 0, kChar = 1, kFloat = 2, kDouble = 3, kInt8 = 4, kInt32 = 5, kInt64 = 6,
  kUInt8 = 7, kOFRecord = 8, kFloat16 = 9, kTensorBuffer = 10, kBFloat16 = 11
};

#define OFQ_STANDALONE_CHECK(cond)                                              \
  if (!(cond)) (std::cerr << "Check failed: " #cond << " " << __FILE__ << ":" << __LINE__ << "\n", std::abort(), std::cerr)
#define CHECK(cond) OFQ_STANDALONE_CHECK(cond)
#define CHECK_EQ(a, b) OFQ_STANDALONE_CHECK((a) == (b))
#define CHECK_GE(a, b) OFQ_STANDALONE_CHECK((a) >= (b))
#define CHECK_GT(a, b) OFQ_STANDALONE_CHECK((a) > (b))
#define CHECK_LT(a, b) OFQ_STANDALONE_CHECK((a) < (b))
#define CHECK_LE(a, b) OFQ_STANDALONE_CHECK((a) <= (b))
#define UNIMPLEMENTED() (std::cerr << "UNIMPLEMENTED " << __FILE__ << ":" << __LINE__ << "\n", std::abort(), std::cerr)

class ShapeView {
 public:
  ShapeView() = default;
  explicit ShapeView(std::vector<int64_t> d) : dims_(std::move(d)) {}
  int64_t NumAxes() const { return (int64_t)dims_.size(); }
  int64_t At(int64_t i) const { return dims_[i]; }
  int64_t Count(int64_t begin, int64_t end) const {
    int64_t c = 1;
    for (int64_t i = begin; i < end; ++i) c *= dims_[i];
    return c;
  }
  int64_t Count(int64_t begin) const { return Count(begin, NumAxes()); }
  int64_t elem_cnt() const { return Count(0); }
  bool operator==(const ShapeView& o) const { return dims_ == o.dims_; }

 private:
  std::vector<int64_t> dims_;
};

// Error::RuntimeError() << "text" converts to a failed Maybe, Maybe<T>::Ok() / a value to a good
// one; IsOk() is what callers test (CHECK_JUST aborts with the message otherwise).
class Error {
 public:
  static Error RuntimeError() { return Error(); }
  template<typename V>
  Error&& operator<<(const V& v) && {
    std::ostringstream os;
    os << v;
    msg_ += os.str();
    return std::move(*this);
  }
  const std::string& msg() const { return msg_; }

 private:
  std::string msg_;
};
template<typename T>
class Maybe;
template<>
class Maybe<void> {
 public:
  static Maybe Ok() { return Maybe(); }
  Maybe(Error&& e) : ok_(false), msg_(e.msg()) {}  // NOLINT
  bool IsOk() const { return ok_; }
  const std::string& error_message() const { return msg_; }

 private:
  Maybe() : ok_(true) {}
  bool ok_;
  std::string msg_;
};
template<>
class Maybe<bool> {
 public:
  Maybe(bool v) : ok_(true), value_(v) {}             // NOLINT
  Maybe(Error&& e) : ok_(false), value_(false), msg_(e.msg()) {}  // NOLINT
  bool IsOk() const { return ok_; }
  bool value() const { return value_; }
  const std::string& error_message() const { return msg_; }

 private:
  bool ok_;
  bool value_;
  std::string msg_;
};
#define CHECK_JUST(expr)                                                       \
  do {                                                                         \
    auto ofq_maybe_ = (expr);                                                  \
    if (!ofq_maybe_.IsOk()) {                                                  \
      std::cerr << "CHECK_JUST failed: " << ofq_maybe_.error_message() << "\n"; \
      std::abort();                                                            \
    }                                                                          \
  } while (0)

#define OFQ_OR_RETURN(cond)                                                              \
  if (!(cond))                                                                           \
  return ::oneflow::Error::RuntimeError() << "Check failed: " #cond " " << __FILE__ << ":" << __LINE__
#define CHECK_OR_RETURN(cond) OFQ_OR_RETURN(cond)
#define CHECK_EQ_OR_RETURN(a, b) OFQ_OR_RETURN((a) == (b))
#define CHECK_GE_OR_RETURN(a, b) OFQ_OR_RETURN((a) >= (b))
#define CHECK_GT_OR_RETURN(a, b) OFQ_OR_RETURN((a) > (b))
#define CHECK_LE_OR_RETURN(a, b) OFQ_OR_RETURN((a) <= (b))
#define CHECK_LT_OR_RETURN(a, b) OFQ_OR_RETURN((a) < (b))
#define UNIMPLEMENTED_THEN_RETURN() \
  return ::oneflow::Error::RuntimeError() << "UNIMPLEMENTED " << __FILE__ << ":" << __LINE__
#define JUST(expr)                               \
  do {                                           \
    auto ofq_just_ = (expr);                     \
    if (!ofq_just_.IsOk()) return ofq_just_;     \
  } while (0)

// oneflow/core/common/shape.h: what the op definitions use of it
class Shape {
 public:
  Shape() = default;
  Shape(std::initializer_list<int64_t> d) : dims_(d) {}
  explicit Shape(std::vector<int64_t> d) : dims_(std::move(d)) {}
  int64_t NumAxes() const { return (int64_t)dims_.size(); }
  int64_t At(int64_t i) const { return dims_[i]; }
  int64_t& operator[](int64_t i) { return dims_[i]; }
  int64_t elem_cnt() const {
    int64_t c = 1;
    for (int64_t d : dims_) c *= d;
    return c;
  }
  bool operator==(const Shape& o) const { return dims_ == o.dims_; }
  bool operator!=(const Shape& o) const { return dims_ != o.dims_; }
  const std::vector<int64_t>& dim_vec() const { return dims_; }

 private:
  std::vector<int64_t> dims_;
};

namespace ep {
class Event {
 public:
  Event() = default;
  virtual ~Event() = default;
  virtual Maybe<bool> QueryDone() = 0;
  virtual Maybe<void> Sync() = 0;
};

class Stream {
 public:
  Stream() = default;
  virtual ~Stream() = default;
  virtual DeviceType device_type() const = 0;
  virtual Maybe<void> Sync() = 0;
  virtual void RecordEvent(Event* event) = 0;
  virtual void WaitEvent(Event*) { UNIMPLEMENTED(); }
  virtual Maybe<void> GetAsyncError() { return Maybe<void>::Ok(); }
  virtual Maybe<void> OnExecutionContextSetup() { return Maybe<void>::Ok(); }
  virtual Maybe<void> OnExecutionContextTeardown() { return Maybe<void>::Ok(); }
  // oneflow/core/ep/include/stream.h:53-56: the device-specific stream is reached by a cast
  template<typename T>
  T* As() {
    return static_cast<T*>(this);
  }
};
}  // namespace ep

namespace user_op {

class Tensor {
 public:
  Tensor(std::vector<int64_t> shape, DataType dt, void* ptr)
      : shape_(std::move(shape)), dtype_(dt), ptr_(ptr) {}
  const ShapeView& shape_view() const { return shape_; }
  DataType data_type() const { return dtype_; }
  template<typename T = void>
  const T* dptr() const { return static_cast<const T*>(ptr_); }
  template<typename T = void>
  T* mut_dptr() { return static_cast<T*>(ptr_); }

 private:
  ShapeView shape_;
  DataType dtype_;
  void* ptr_;
};

struct AttrValue {
  int64_t i = 0;
  double f = 0;
  bool b = false;
  std::string s;
};

class KernelComputeContext {
 public:
  virtual ~KernelComputeContext() = default;
  Tensor* Tensor4ArgNameAndIndex(const std::string& name, int32_t index) {
    auto it = tensors_.find({name, index});
    return it == tensors_.end() ? nullptr : it->second.get();
  }
  bool has_input(const std::string& name, int32_t index) const {
    return tensors_.count({name, index}) != 0;
  }
  template<typename T>
  T Attr(const std::string& name) const;
  ep::Stream* stream() { return stream_; }

  // number of tensors bound to a variadic argument (user_op::KernelComputeContext::input_size)
  int32_t input_size(const std::string& name) const {
    int32_t n = 0;
    while (tensors_.count({name, n}) != 0) ++n;
    return n;
  }

  // test-side helpers
  void AddTensor(const std::string& name, std::vector<int64_t> shape, DataType dt, void* ptr,
                 int32_t index = 0) {
    tensors_[{name, index}] = std::make_unique<Tensor>(std::move(shape), dt, ptr);
  }
  std::map<std::string, AttrValue> attrs;
  ep::Stream* stream_ = nullptr;

 private:
  std::map<std::pair<std::string, int32_t>, std::unique_ptr<Tensor>> tensors_;
};
template<> inline int32_t KernelComputeContext::Attr<int32_t>(const std::string& n) const { return (int32_t)attrs.at(n).i; }
template<> inline int64_t KernelComputeContext::Attr<int64_t>(const std::string& n) const { return attrs.at(n).i; }
template<> inline bool KernelComputeContext::Attr<bool>(const std::string& n) const { return attrs.at(n).b; }
template<> inline float KernelComputeContext::Attr<float>(const std::string& n) const { return (float)attrs.at(n).f; }
template<> inline double KernelComputeContext::Attr<double>(const std::string& n) const { return attrs.at(n).f; }
template<> inline std::string KernelComputeContext::Attr<std::string>(const std::string& n) const { return attrs.at(n).s; }

// oneflow/core/framework/tensor_desc.h: shape and dtype of an argument
class TensorDesc {
 public:
  TensorDesc() = default;
  TensorDesc(Shape s, DataType d) : shape_(std::move(s)), dtype_(d) {}
  const Shape& shape() const { return shape_; }
  DataType data_type() const { return dtype_; }

 private:
  Shape shape_;
  DataType dtype_ = kInvalidDataType;
};

// oneflow/core/framework/infer_util.h:35-90 (user_op::InferContext): inputs by (name, index),
// outputs set by the op definition's inference functions.  `shapes` / `dtypes` (index 0 by name)
// serve the kernels' tmp_buffer sizing; `in` / `out` (by name and index) the op definitions.
class InferContext {
 public:
  virtual ~InferContext() = default;
  std::map<std::string, std::vector<int64_t>> shapes;
  std::map<std::string, DataType> dtypes;
  ShapeView InputShape(const std::string& name, int32_t index) const {
    auto it = in.find({name, index});
    if (it != in.end()) return ShapeView(it->second.shape().dim_vec());
    return ShapeView(shapes.at(name));
  }
  DataType InputDType(const std::string& name, int32_t index) const {
    auto it = in.find({name, index});
    return it != in.end() ? it->second.data_type() : dtypes.at(name);
  }
  std::map<std::string, AttrValue> attrs;
  template<typename T>
  T Attr(const std::string& name) const;

  std::map<std::pair<std::string, int32_t>, TensorDesc> in, out;
  void AddInput(const std::string& name, int32_t index, std::vector<int64_t> shape, DataType dt) {
    in[{name, index}] = TensorDesc(Shape(std::move(shape)), dt);
  }
  const TensorDesc& InputTensorDesc(const std::string& name, int32_t index) const {
    return in.at({name, index});
  }
  bool has_input(const std::string& name, int32_t index) const { return in.count({name, index}) != 0; }
  int32_t input_size(const std::string& name) const {
    int32_t n = 0;
    while (in.count({name, n}) != 0) ++n;
    return n;
  }
  void SetOutputShape(const std::string& name, int32_t index, const Shape& shape) {
    out[{name, index}] = TensorDesc(shape, out[{name, index}].data_type());
  }
  void SetOutputDType(const std::string& name, int32_t index, DataType dt) {
    out[{name, index}] = TensorDesc(out[{name, index}].shape(), dt);
  }
};
template<> inline bool InferContext::Attr<bool>(const std::string& n) const { return attrs.at(n).b; }
template<> inline int32_t InferContext::Attr<int32_t>(const std::string& n) const { return (int32_t)attrs.at(n).i; }
template<> inline int64_t InferContext::Attr<int64_t>(const std::string& n) const { return attrs.at(n).i; }
template<> inline double InferContext::Attr<double>(const std::string& n) const { return attrs.at(n).f; }
template<> inline std::string InferContext::Attr<std::string>(const std::string& n) const { return attrs.at(n).s; }
template<> inline DataType InferContext::Attr<DataType>(const std::string& n) const { return (DataType)attrs.at(n).i; }

class OpKernelState {};
class OpKernelCache {};

class OpKernel {
 public:
  virtual ~OpKernel() = default;
  virtual void Compute(KernelComputeContext* ctx, OpKernelState*, const OpKernelCache*) const {
    Compute(ctx);
  }
  virtual void Compute(KernelComputeContext*) const {}
  virtual bool AlwaysComputeWhenAllOutputsEmpty() const = 0;
};

// predicates: only what is needed to record and evaluate (device, dtype-of-arg) matches
struct KernelRegContext {
  DeviceType device;
  std::map<std::string, DataType> arg_dtypes;
};
using IsMatchedHob = std::function<bool(const KernelRegContext&)>;
struct HobDeviceTypeT {};
struct HobDataTypeT { std::string name; };
inline HobDeviceTypeT HobDeviceType() { return {}; }
inline HobDataTypeT HobDataType(const std::string& name, int) { return {name}; }
inline IsMatchedHob operator==(HobDeviceTypeT, DeviceType d) {
  return [d](const KernelRegContext& c) { return c.device == d; };
}
inline IsMatchedHob operator==(HobDataTypeT h, DataType t) {
  return [h, t](const KernelRegContext& c) {
    auto it = c.arg_dtypes.find(h.name);
    return it != c.arg_dtypes.end() && it->second == t;
  };
}
inline IsMatchedHob operator&&(IsMatchedHob a, IsMatchedHob b) {
  return [a, b](const KernelRegContext& c) { return a(c) && b(c); };
}

constexpr int32_t kKernelPriorityFallback = -10;
constexpr int32_t kKernelPriorityDefault = 0;
constexpr int32_t kKernelPriorityOptimized = 10;

struct KernelRegistration {
  std::string op_type_name;
  std::function<std::unique_ptr<OpKernel>()> create;
  IsMatchedHob matched;
  std::function<size_t(InferContext*)> infer_tmp_size;
  int32_t priority = kKernelPriorityDefault;
};
inline std::vector<KernelRegistration>& KernelRegistry() {
  static std::vector<KernelRegistration> r;
  return r;
}
class OpKernelRegistry {
 public:
  explicit OpKernelRegistry(const std::string& name) { reg_.op_type_name = name; }
  template<typename K>
  OpKernelRegistry& SetCreateFn() {
    reg_.create = [] { return std::unique_ptr<OpKernel>(new K()); };
    return *this;
  }
  OpKernelRegistry& SetIsMatchedHob(IsMatchedHob h) {
    reg_.matched = std::move(h);
    return *this;
  }
  OpKernelRegistry& SetInferTmpSizeFn(std::function<size_t(InferContext*)> f) {
    reg_.infer_tmp_size = std::move(f);
    return *this;
  }
  OpKernelRegistry& SetPriority(int32_t p) {
    reg_.priority = p;
    return *this;
  }
  const KernelRegistration& Finish() const { return reg_; }

 private:
  KernelRegistration reg_;
};
struct Registrar {
  Registrar(const OpKernelRegistry& r) { KernelRegistry().push_back(r.Finish()); }  // NOLINT
};

}  // namespace user_op

#define OFQ_CAT_(a, b) a##b
#define OFQ_CAT(a, b) OFQ_CAT_(a, b)
#define REGISTER_USER_KERNEL(name) \
  static ::oneflow::user_op::Registrar OFQ_CAT(g_ofq_registrar_, __COUNTER__) = ::oneflow::user_op::OpKernelRegistry(name)

}  // namespace oneflow
