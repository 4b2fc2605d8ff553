// mace_hip_delegator.h -- C++ host side above the C ABI (mace_hip.h).
//
// Header-only mirror of the reference interfaces this path plugs into, with the same names,
// argument meaning and error behaviour, so that a MACE maintainer can see the drop-in without
// building MACE:
//   * delegator::Gemm / delegator::Gemv / delegator::Conv2d virtual signatures
//     (mace/ops/delegator/gemm.h:35-70, gemv.h:27-46, conv_2d.h:60-82),
//   * DelegatorInfo keys, OpDelegatorRegistry::Register / GetCreator with the reference's
//     fallback rule (mace/core/registry/op_delegator_registry.cc:39-103),
//   * the shape derivation and dispatch of MatMulOp, FullyConnectedOp and the quantized 1x1
//     Conv2dOp (mace/ops/matmul.cc:55-83,110-215,397-483; fully_connected.cc:82-121,141-179;
//     conv_2d.cc:201-318; arm/base/conv_2d_1x1.cc:27-72).
// Everything lives in namespace mace_hip so the header can sit next to the real MACE headers.
// In a MACE tree the hip:: classes derive from mace::ops::delegator::* instead and are
// registered under the keys the ops ask for.
//
// Contract violations the reference handles with MACE_CHECK (process abort) are reported as
// MaceStatus::MACE_INVALID_ARGS here.
#ifndef MACE_HIP_DELEGATOR_H_
#define MACE_HIP_DELEGATOR_H_

#include <algorithm>
#include <cstdint>
#include <cstdlib>
#include <functional>
#include <initializer_list>
#include <cmath>
#include <memory>
#include <numeric>
#include <sstream>
#include <type_traits>
#include <string>
#include <unordered_map>
#include <vector>

#include "mace_hip.h"

namespace mace_hip {

typedef int64_t index_t;

// include/mace/public/mace.h:244-250
enum class MaceStatus {
  MACE_SUCCESS = 0,
  MACE_INVALID_ARGS = 1,
  MACE_OUT_OF_RESOURCES = 2,
  MACE_UNSUPPORTED = 3,
  MACE_RUNTIME_ERROR = 4
};
inline MaceStatus ToStatus(int code) { return static_cast<MaceStatus>(code); }

enum DataType { DT_INVALID = 0, DT_FLOAT = 1, DT_UINT8 = 2, DT_INT32 = 4 };  // mace.proto
enum RuntimeType { RT_CPU = 0, RT_OPENCL = 2 };            // include/mace/public/mace.h
enum ImplType { REF = 0, NEON };                            // mace/core/ops/op_delegator.h:25-28
const ImplType kCpuImplType = ImplType::REF;                // :30-34 on a non-NEON host
enum MatrixMajor { RowMajor = MACE_HIP_ROW_MAJOR, ColMajor = MACE_HIP_COL_MAJOR };
// mace/ops/common/activation_type.h; the kernels of this library apply the first three
enum ActivationType { NOOP = MACE_HIP_ACT_NOOP, RELU = MACE_HIP_ACT_RELU,
                      RELUX = MACE_HIP_ACT_RELUX, PRELU = 3, TANH = 4, SIGMOID = 5, LEAKYRELU = 6,
                      ELU = 7, HARDSIGMOID = 8 };
// mace/ops/common/activation_type.h StringToActivationType; false for a name it does not know
inline bool StringToActivationType(const std::string &name, ActivationType *type) {
  static const char *const names[] = {"NOOP", "RELU", "RELUX", "PRELU", "TANH", "SIGMOID",
                                      "LEAKYRELU", "ELU", "HARDSIGMOID"};
  for (int i = 0; i < 9; ++i)
    if (name == names[i]) { *type = static_cast<ActivationType>(i); return true; }
  return false;
}

template <typename T> struct DataTypeToEnum;
template <> struct DataTypeToEnum<float> { static const DataType value = DT_FLOAT; };
template <> struct DataTypeToEnum<uint8_t> { static const DataType value = DT_UINT8; };
template <> struct DataTypeToEnum<int32_t> { static const DataType value = DT_INT32; };

// The part of mace::Tensor the delegators use (mace/core/tensor.h:147-256): typed data
// pointer, shape, scale / zero point, weight flag.  Memory is owned by the caller; it is host
// memory unless on_device is set.
class Tensor {
 public:
  Tensor() = default;
  Tensor(void *data, DataType dtype, std::vector<index_t> shape, float scale = 0.f,
         int32_t zero_point = 0, bool is_weight = false, bool on_device = false)
      : data_(data), dtype_(dtype), shape_(std::move(shape)), scale_(scale),
        zero_point_(zero_point), is_weight_(is_weight), on_device_(on_device) {}
  template <typename T> const T *data() const { return static_cast<const T *>(data_); }
  template <typename T> T *mutable_data() { return static_cast<T *>(data_); }
  const std::vector<index_t> &shape() const { return shape_; }
  index_t dim_size() const { return static_cast<index_t>(shape_.size()); }
  index_t dim(index_t i) const { return shape_[i]; }
  index_t size() const {
    return std::accumulate(shape_.begin(), shape_.end(), index_t(1), std::multiplies<index_t>());
  }
  DataType dtype() const { return dtype_; }
  float scale() const { return scale_; }
  int32_t zero_point() const { return zero_point_; }
  void SetScale(float s) { scale_ = s; }
  void SetZeroPoint(int32_t z) { zero_point_ = z; }
  bool is_weight() const { return is_weight_; }
  bool on_device() const { return on_device_; }
  // The caller allocates; Resize only records the shape and checks it fits (capacity in
  // elements, 0 = unchecked).
  MaceStatus Resize(const std::vector<index_t> &shape, index_t capacity = 0) {
    shape_ = shape;
    if (capacity > 0 && size() > capacity) return MaceStatus::MACE_OUT_OF_RESOURCES;
    return MaceStatus::MACE_SUCCESS;
  }

 private:
  void *data_ = nullptr;
  DataType dtype_ = DT_INVALID;
  std::vector<index_t> shape_;
  float scale_ = 0.f;
  int32_t zero_point_ = 0;
  bool is_weight_ = false;
  bool on_device_ = false;
};

// mace/core/ops/op_context.h:24-41: what an op hands to its delegators.  Here it carries the
// library context (stream + scratch arena) instead of a CPU runtime with a thread pool.
class OpContext {
 public:
  explicit OpContext(mace_hip_ctx *ctx) : ctx_(ctx) {}
  mace_hip_ctx *hip() const { return ctx_; }

 private:
  mace_hip_ctx *ctx_;
};

struct DelegatorParam {            // mace/core/ops/op_delegator.h:36-40
  DelegatorParam() = default;
  virtual ~DelegatorParam() = default;
};
class OpDelegator {                // mace/core/ops/op_delegator.h:42-55
 public:
  explicit OpDelegator(const DelegatorParam &) {}
  virtual ~OpDelegator() = default;
  template <class DerivedType, class ParamType>
  static std::unique_ptr<OpDelegator> DefaultCreator(const DelegatorParam &param) {
    return std::unique_ptr<OpDelegator>(
        new DerivedType(static_cast<const ParamType &>(param)));
  }
};

// ---- registry (mace/core/registry/op_delegator_registry.{h,cc}) --------------------------------
typedef std::function<std::unique_ptr<OpDelegator>(const DelegatorParam &)> DelegatorCreator;
static const char *const kDefaultTag = "general";

struct DelegatorInfo {
  DelegatorInfo(const char *name, DataType dt, RuntimeType rt, ImplType impl,
                const char *in_tag = kDefaultTag)
      : delegator_name(name), data_type(dt), runtime(rt), impl_type(impl), tag(in_tag) {}
  std::string ToString() const {      // op_delegator_registry.cc:39-44
    std::stringstream ss;
    ss << delegator_name << "_" << data_type << "_" << runtime << "_" << impl_type << "_" << tag;
    return ss.str();
  }
  bool operator==(const DelegatorInfo &o) const {
    return runtime == o.runtime && impl_type == o.impl_type && data_type == o.data_type &&
           delegator_name == o.delegator_name && tag == o.tag;
  }
  std::string delegator_name;
  DataType data_type;
  RuntimeType runtime;
  ImplType impl_type;
  std::string tag;
};

class OpDelegatorRegistry {
 public:
  // op_delegator_registry.cc:52-58: a duplicate key is a CHECK failure in the reference
  MaceStatus Register(const DelegatorInfo &key, DelegatorCreator creator) {
    if (registry_.count(key.ToString()) > 0) return MaceStatus::MACE_INVALID_ARGS;
    registry_[key.ToString()] = std::move(creator);
    return MaceStatus::MACE_SUCCESS;
  }
  // op_delegator_registry.cc:64-103: exact key, then NEON -> general tag -> REF (+tag) ->
  // REF general.  The reference LOG(FATAL)s when nothing matches; an empty creator here.
  DelegatorCreator GetCreator(const DelegatorInfo &key) const {
    auto find = [&](const DelegatorInfo &k) { return registry_.find(k.ToString()); };
    auto it = find(key);
    if (it != registry_.end()) return it->second;
    DelegatorInfo info = key;
    if (key.impl_type == ImplType::NEON) {
      if (info.tag != kDefaultTag) {
        info.tag = kDefaultTag;
        if ((it = find(info)) != registry_.end()) return it->second;
        info.tag = key.tag;
      }
      info.impl_type = ImplType::REF;
      if ((it = find(info)) != registry_.end()) return it->second;
    }
    if (info.tag != kDefaultTag) {
      info.tag = kDefaultTag;
      if ((it = find(info)) != registry_.end()) return it->second;
    }
    return DelegatorCreator();
  }

 private:
  std::unordered_map<std::string, DelegatorCreator> registry_;
};

#define MACE_HIP_DELEGATOR_KEY(name, rt, DT, impl) \
  ::mace_hip::DelegatorInfo(#name, ::mace_hip::DataTypeToEnum<DT>::value, rt, impl)
#define MACE_HIP_DELEGATOR_KEY_EX(name, rt, DT, impl, tag) \
  ::mace_hip::DelegatorInfo(#name, ::mace_hip::DataTypeToEnum<DT>::value, rt, impl, #tag)
#define MACE_HIP_REGISTER_DELEGATOR(registry, class_name, param_name, key) \
  (registry)->Register(key, ::mace_hip::OpDelegator::DefaultCreator<class_name, param_name>)

enum Padding { VALID = 0, SAME = 1, FULL = 2 };   // mace/ops/common/conv_pool_2d_util.h

// ---- abstract delegators ---------------------------------------------------------------------------
namespace delegator {

struct GemmParam : public DelegatorParam {     // mace/ops/delegator/gemm.h:28-33
  explicit GemmParam(const bool should_cache_pack = false)
      : should_cache_pack_(should_cache_pack) {}
  const bool should_cache_pack_;
};

class Gemm : public OpDelegator {              // mace/ops/delegator/gemm.h:35-70
 public:
  explicit Gemm(const GemmParam &param) : OpDelegator(param) {}
  virtual MaceStatus Compute(const OpContext *context, const Tensor *lhs, const Tensor *rhs,
                             const index_t batch, const index_t rows, const index_t cols,
                             const index_t depth, const MatrixMajor lhs_major,
                             const MatrixMajor rhs_major, const MatrixMajor output_major,
                             const bool lhs_batched, const bool rhs_batched,
                             Tensor *output) = 0;
  // Original matrix before transpose has row-major
  virtual MaceStatus Compute(const OpContext *context, const Tensor *lhs, const Tensor *rhs,
                             const index_t batch, const index_t lhs_rows,
                             const index_t lhs_cols, const index_t rhs_rows,
                             const index_t rhs_cols, const bool transpose_lhs,
                             const bool transpose_rhs, const bool transpose_out,
                             const bool lhs_batched, const bool rhs_batched,
                             Tensor *output) = 0;
};

class Gemv : public OpDelegator {              // mace/ops/delegator/gemv.h:27-46
 public:
  explicit Gemv(const DelegatorParam &param) : OpDelegator(param) {}
  // Always row-major after transpose
  virtual MaceStatus Compute(const OpContext *context, const Tensor *lhs, const Tensor *rhs,
                             const Tensor *bias, const index_t batch,
                             const index_t lhs_height, const index_t lhs_width,
                             const bool lhs_batched, const bool rhs_batched,
                             Tensor *output) = 0;
};

struct Conv2dParam : public DelegatorParam {   // mace/ops/delegator/conv_2d.h:46-58
  explicit Conv2dParam(const std::vector<int> &strides = {1, 1},
                       const std::vector<int> &dilations = {1, 1},
                       const std::vector<int> &paddings = {},
                       const Padding padding_type = SAME)
      : strides_(strides), dilations_(dilations), paddings_(paddings),
        padding_type_(padding_type) {}
  const std::vector<int> strides_;
  const std::vector<int> dilations_;
  const std::vector<int> paddings_;   // empty: derive from padding_type_
  const Padding padding_type_;
};
class Conv2d : public OpDelegator {            // mace/ops/delegator/conv_2d.h:60-82
 public:
  explicit Conv2d(const Conv2dParam &param)
      : OpDelegator(param), strides_(param.strides_), dilations_(param.dilations_),
        paddings_(param.paddings_), padding_type_(param.padding_type_) {}
  virtual MaceStatus Compute(const OpContext *context, const Tensor *input,
                             const Tensor *filter, Tensor *output) = 0;

 protected:
  const std::vector<int> strides_;
  const std::vector<int> dilations_;
  const std::vector<int> paddings_;
  const Padding padding_type_;
};

}  // namespace delegator

// Where the operands of a call live.  The C ABI has two families of entry points -- device
// pointers, ordered on the context's stream, and host pointers, staged and synchronous -- and a
// call must go to one of them as a whole: every operand has to live where the output does.  A mix
// (say a device output with a weight still in host memory, the natural state of a half-migrated
// integration) would hand a host address to a kernel, so it is refused before anything is launched.
inline bool SamePlacement(const Tensor *output, std::initializer_list<const Tensor *> inputs) {
  for (const Tensor *t : inputs)
    if (t != nullptr && t->on_device() != output->on_device()) return false;
  return true;
}

// A constant operand kept resident across calls.  MACE's delegators may keep a packed copy of a
// weight (GemmParam::should_cache_pack_ with Tensor::is_weight(), mace/ops/delegator/gemm.h:28-33,
// mace/ops/arm/base/gemm.cc:560-576, which then stops reading the original).  Counterpart: an
// operand that is_weight() is registered with the library context once per op instance --
//   * in device memory: its repacked uint8 panel and row sums are kept across Run() calls;
//   * in host memory: it is uploaded once, and the host-pointer entry points then move only the
//     activations (the registered copy also keeps its panel and sums).
// A weight whose buffer moves is registered afresh; Refresh() re-registers one whose contents the
// caller has changed.  The registration ends with the op (or when the weight moves): the caches are
// keyed by address, and once the weight's buffer has been freed the allocator may hand the same
// address to an activation tensor, which must not find a stale copy.  The op must be destroyed
// before its library context is.
class WeightRegistration {
 public:
  WeightRegistration() = default;
  WeightRegistration(const WeightRegistration &) = delete;
  WeightRegistration &operator=(const WeightRegistration &) = delete;
  ~WeightRegistration() { Release(); }
  void Note(const OpContext *context, const Tensor *t, size_t bytes) {
    if (t == nullptr || !t->is_weight() || bytes == 0) return;
    const void *ptr = t->data<uint8_t>();
    if (ptr == registered_ && context->hip() == ctx_ && bytes == bytes_ && t->on_device() == device_)
      return;
    Release();
    const int rc = t->on_device() ? mace_hip_weight_register(context->hip(), ptr, bytes)
                                  : mace_hip_host_weight_register(context->hip(), ptr, bytes);
    if (rc == MACE_HIP_SUCCESS) {
      registered_ = ptr;
      ctx_ = context->hip();
      bytes_ = bytes;
      device_ = t->on_device();
    }
  }
  // the caller has written new values into the registered weight
  void Refresh() {
    if (registered_ == nullptr) return;
    if (device_) (void)mace_hip_weight_register(ctx_, registered_, bytes_);
    else (void)mace_hip_host_weight_register(ctx_, registered_, bytes_);
  }
  void Release() {
    if (registered_ != nullptr) {
      if (device_) (void)mace_hip_weight_unregister(ctx_, registered_);
      else (void)mace_hip_host_weight_unregister(ctx_, registered_);
    }
    registered_ = nullptr;
    ctx_ = nullptr;
  }

 private:
  const void *registered_ = nullptr;
  mace_hip_ctx *ctx_ = nullptr;
  size_t bytes_ = 0;
  bool device_ = false;
};

// ---- the GPU delegators --------------------------------------------------------------------------------
namespace hip {

template <typename T> class Gemm;
template <>
class Gemm<float> : public delegator::Gemm {   // replaces ref::Gemm<float> / arm::Gemm<float>
 public:
  explicit Gemm(const delegator::GemmParam &param)
      : delegator::Gemm(param), should_cache_pack_(param.should_cache_pack_) {}
  MaceStatus Compute(const OpContext *context, const Tensor *lhs, const Tensor *rhs,
                     const index_t batch, const index_t rows, const index_t cols,
                     const index_t depth, const MatrixMajor lhs_major,
                     const MatrixMajor rhs_major, const MatrixMajor output_major,
                     const bool lhs_batched, const bool rhs_batched,
                     Tensor *output) override {
    if (!SamePlacement(output, {lhs, rhs})) return MaceStatus::MACE_INVALID_ARGS;
    // mace/ops/arm/base/gemm.cc:560-576: with should_cache_pack_, the weight side (the left one
    // first) is kept across calls unless it differs per batch
    if (should_cache_pack_) {
      if (lhs->is_weight() && (!lhs_batched || batch == 1))
        cache_.Note(context, lhs, sizeof(float) * static_cast<size_t>(rows * depth));
      else if (rhs->is_weight() && (!rhs_batched || batch == 1))
        cache_.Note(context, rhs, sizeof(float) * static_cast<size_t>(depth * cols));
    }
    auto fn = output->on_device() ? mace_hip_gemm_f32 : mace_hip_gemm_f32_host;
    return ToStatus(fn(context->hip(), lhs->data<float>(), rhs->data<float>(), batch, rows,
                       cols, depth, lhs_major, rhs_major, output_major, lhs_batched,
                       rhs_batched, output->mutable_data<float>()));
  }
  MaceStatus Compute(const OpContext *context, const Tensor *lhs, const Tensor *rhs,
                     const index_t batch, const index_t lhs_rows, const index_t lhs_cols,
                     const index_t rhs_rows, const index_t rhs_cols, const bool transpose_lhs,
                     const bool transpose_rhs, const bool transpose_out,
                     const bool lhs_batched, const bool rhs_batched,
                     Tensor *output) override {
    // mace/ops/ref/gemm.cc:122-145
    const index_t rows = transpose_lhs ? lhs_cols : lhs_rows;
    const index_t depth = transpose_lhs ? lhs_rows : lhs_cols;
    const index_t cols = transpose_rhs ? rhs_rows : rhs_cols;
    const index_t depth2 = transpose_rhs ? rhs_cols : rhs_rows;
    if (depth != depth2) return MaceStatus::MACE_INVALID_ARGS;
    return Compute(context, lhs, rhs, batch, rows, cols, depth,
                   transpose_lhs ? ColMajor : RowMajor, transpose_rhs ? ColMajor : RowMajor,
                   transpose_out ? ColMajor : RowMajor, lhs_batched, rhs_batched, output);
  }

 private:
  const bool should_cache_pack_;
  WeightRegistration cache_;
};

template <typename T> class Gemv;
template <>
class Gemv<float> : public delegator::Gemv {   // replaces ref::Gemv<float> / arm::Gemv<float>
 public:
  explicit Gemv(const DelegatorParam &param) : delegator::Gemv(param) {}
  MaceStatus Compute(const OpContext *context, const Tensor *lhs, const Tensor *rhs,
                     const Tensor *bias, const index_t batch, const index_t lhs_height,
                     const index_t lhs_width, const bool lhs_batched, const bool rhs_batched,
                     Tensor *output) override {
    return ComputeFused(context, lhs, rhs, bias, batch, lhs_height, lhs_width, lhs_batched,
                        rhs_batched, NOOP, 0.f, output);
  }
  // Compute followed by the Activation delegator as FullyConnectedOp runs it
  // (mace/ops/fully_connected.cc:108-121), applied as the sums are stored.
  MaceStatus ComputeFused(const OpContext *context, const Tensor *lhs, const Tensor *rhs,
                          const Tensor *bias, const index_t batch, const index_t lhs_height,
                          const index_t lhs_width, const bool lhs_batched, const bool rhs_batched,
                          ActivationType activation, float max_limit, Tensor *output) {
    if (!SamePlacement(output, {lhs, rhs, bias})) return MaceStatus::MACE_INVALID_ARGS;
    // a constant weight matrix (and bias) stays on the GPU between calls
    if (!lhs_batched) weight_.Note(context, lhs, sizeof(float) * static_cast<size_t>(lhs_height * lhs_width));
    if (bias) bias_.Note(context, bias, sizeof(float) * static_cast<size_t>(lhs_height));
    auto fn = output->on_device() ? mace_hip_gemv_f32_act : mace_hip_gemv_f32_act_host;
    return ToStatus(fn(context->hip(), lhs->data<float>(), rhs->data<float>(),
                       bias ? bias->data<float>() : nullptr, batch, lhs_height, lhs_width,
                       lhs_batched, rhs_batched, activation, max_limit,
                       output->mutable_data<float>()));
  }

 private:
  WeightRegistration weight_, bias_;
};
// Replaces ref::q8::Gemv<uint8_t> (requant_mode REF) / arm::q8::Gemv<uint8_t> (NEON).
template <>
class Gemv<uint8_t> : public delegator::Gemv {
 public:
  explicit Gemv(const DelegatorParam &param, int requant_mode = MACE_HIP_REQUANT_NEON)
      : delegator::Gemv(param), requant_mode_(requant_mode) {}
  MaceStatus Compute(const OpContext *context, const Tensor *lhs, const Tensor *rhs,
                     const Tensor *bias, const index_t batch, const index_t lhs_height,
                     const index_t lhs_width, const bool lhs_batched, const bool rhs_batched,
                     Tensor *output) override {
    if (!SamePlacement(output, {lhs, rhs, bias})) return MaceStatus::MACE_INVALID_ARGS;
    if (!lhs_batched) weight_.Note(context, lhs, static_cast<size_t>(lhs_height * lhs_width));
    if (bias) bias_.Note(context, bias, sizeof(int32_t) * static_cast<size_t>(lhs_height));
    auto fn = output->on_device() ? mace_hip_gemv_q8_u8 : mace_hip_gemv_q8_u8_host;
    return ToStatus(fn(context->hip(), lhs->data<uint8_t>(), rhs->data<uint8_t>(),
                       bias ? bias->data<int32_t>() : nullptr, batch, lhs_height, lhs_width,
                       lhs_batched, rhs_batched, lhs->zero_point(), rhs->zero_point(),
                       lhs->scale(), rhs->scale(), output->scale(), output->zero_point(),
                       requant_mode_, output->mutable_data<uint8_t>()));
  }

 private:
  int requant_mode_;
  WeightRegistration weight_, bias_;
};
template <>
class Gemv<int32_t> : public delegator::Gemv {   // replaces ref::q8::Gemv<int32_t>
 public:
  explicit Gemv(const DelegatorParam &param) : delegator::Gemv(param) {}
  MaceStatus Compute(const OpContext *context, const Tensor *lhs, const Tensor *rhs,
                     const Tensor *bias, const index_t batch, const index_t lhs_height,
                     const index_t lhs_width, const bool lhs_batched, const bool rhs_batched,
                     Tensor *output) override {
    if (!SamePlacement(output, {lhs, rhs, bias})) return MaceStatus::MACE_INVALID_ARGS;
    if (!lhs_batched) weight_.Note(context, lhs, static_cast<size_t>(lhs_height * lhs_width));
    if (bias) bias_.Note(context, bias, sizeof(int32_t) * static_cast<size_t>(lhs_height));
    auto fn = output->on_device() ? mace_hip_gemv_q8_i32 : mace_hip_gemv_q8_i32_host;
    return ToStatus(fn(context->hip(), lhs->data<uint8_t>(), rhs->data<uint8_t>(),
                       bias ? bias->data<int32_t>() : nullptr, batch, lhs_height, lhs_width,
                       lhs_batched, rhs_batched, lhs->zero_point(), rhs->zero_point(),
                       output->mutable_data<int32_t>()));
  }

 private:
  WeightRegistration weight_, bias_;
};

// The float Conv2d delegator, NCHW input {n, cin, h, w}, OIHW filter {cout, cin, kh, kw}, output
// {n, cout, oh, ow}.  The output shape and padding come from the delegator's parameters exactly
// as in ref::Conv2d / arm::Conv2dBase (mace/ops/ref/conv_2d.cc:44-66,
// mace/ops/arm/base/conv_2d.cc:27-50): from the padding type, or from explicit paddings with the
// FLOOR rule.  The geometry Conv2dOp hands to Conv2dK1x1 -- 1x1 filter, stride 1, dilation 1
// (mace/ops/conv_2d.cc:101-105) -- runs on the GPU, a padded input included (the reference copies
// it into a zero-padded tensor first, mace/ops/arm/base/conv_2d_1x1.cc:37-60).  Every other
// geometry returns MACE_UNSUPPORTED without touching the output: in a MACE tree that branch is
// `return ref::Conv2d<float>::Compute(...)`.
// ComputeFused additionally applies the op's BiasAdd and Activation (mace/ops/conv_2d.cc:171-173)
// as the result is stored; Compute (the virtual of the interface) is ComputeFused without them.
template <typename T> class Conv2d;
template <>
class Conv2d<float> : public delegator::Conv2d {
 public:
  explicit Conv2d(const delegator::Conv2dParam &param) : delegator::Conv2d(param) {}
  MaceStatus Compute(const OpContext *context, const Tensor *input, const Tensor *filter,
                     Tensor *output) override {
    return ComputeFused(context, input, filter, nullptr, NOOP, 0.f, output);
  }
  MaceStatus ComputeFused(const OpContext *context, const Tensor *input, const Tensor *filter,
                          const Tensor *bias, ActivationType activation, float max_limit,
                          Tensor *output) {
    if (input->dim_size() != 4 || filter->dim_size() != 4 || filter->dim(1) != input->dim(1))
      return MaceStatus::MACE_INVALID_ARGS;
    if (strides_.size() != 2 || dilations_.size() != 2) return MaceStatus::MACE_INVALID_ARGS;
    if (bias && (bias->dim_size() != 1 || bias->dim(0) != filter->dim(0)))
      return MaceStatus::MACE_INVALID_ARGS;
    int64_t out_h = 0, out_w = 0;
    int pads[2] = {0, 0};
    if (paddings_.empty()) {
      MaceStatus st = ToStatus(mace_hip_calc_padding_and_output_size(
          input->dim(2), input->dim(3), filter->dim(2), filter->dim(3), dilations_[0],
          dilations_[1], strides_[0], strides_[1], padding_type_, &out_h, &out_w, &pads[0],
          &pads[1]));
      if (st != MaceStatus::MACE_SUCCESS) return st;
    } else {
      if (paddings_.size() != 2 || strides_[0] <= 0 || strides_[1] <= 0)
        return MaceStatus::MACE_INVALID_ARGS;
      pads[0] = paddings_[0];
      pads[1] = paddings_[1];
      const index_t kh = (filter->dim(2) - 1) * dilations_[0] + 1;
      const index_t kw = (filter->dim(3) - 1) * dilations_[1] + 1;
      out_h = static_cast<int64_t>(std::floor(1.0 * (input->dim(2) + pads[0] - kh) / strides_[0]) + 1);
      out_w = static_cast<int64_t>(std::floor(1.0 * (input->dim(3) + pads[1] - kw) / strides_[1]) + 1);
    }
    const bool k1x1 = filter->dim(2) == 1 && filter->dim(3) == 1 && strides_[0] == 1 &&
                      strides_[1] == 1 && dilations_[0] == 1 && dilations_[1] == 1;
    if (!k1x1) return MaceStatus::MACE_UNSUPPORTED;   // stays with ref::Conv2d
    if (!SamePlacement(output, {input, filter, bias})) return MaceStatus::MACE_INVALID_ARGS;
    MaceStatus st = output->Resize({input->dim(0), filter->dim(0), out_h, out_w});
    if (st != MaceStatus::MACE_SUCCESS) return st;
    filter_.Note(context, filter, sizeof(float) * static_cast<size_t>(filter->size()));
    if (bias) bias_.Note(context, bias, sizeof(float) * static_cast<size_t>(bias->size()));
    auto fn = output->on_device() ? mace_hip_conv2d_f32_nchw : mace_hip_conv2d_f32_nchw_host;
    return ToStatus(fn(context->hip(), input->data<float>(), filter->data<float>(),
                       bias ? bias->data<float>() : nullptr, input->dim(0), input->dim(1),
                       input->dim(2), input->dim(3), filter->dim(0), 1, 1, 1, 1, 1, 1, pads[0],
                       pads[1], activation, max_limit, output->mutable_data<float>()));
  }

 private:
  WeightRegistration filter_, bias_;
};
// The same delegator under the name the NEON build registers for the K1x1 tag
// (mace/ops/arm/base/conv_2d_1x1.cc:74-88).
template <typename T> class Conv2dK1x1;
template <>
class Conv2dK1x1<float> : public Conv2d<float> {
 public:
  explicit Conv2dK1x1(const delegator::Conv2dParam &param) : Conv2d<float>(param) {}
};

// mace/ops/registry/op_delegators_registry.cc:87-143 registers ref:: and arm:: delegators; this
// registers the GPU ones under the keys the ops ask for (kCpuImplType), in their place.
inline MaceStatus RegisterAllHipDelegators(OpDelegatorRegistry *registry) {
  MaceStatus st = MACE_HIP_REGISTER_DELEGATOR(
      registry, Gemm<float>, delegator::GemmParam,
      MACE_HIP_DELEGATOR_KEY(Gemm, RT_CPU, float, kCpuImplType));
  if (st != MaceStatus::MACE_SUCCESS) return st;
  st = MACE_HIP_REGISTER_DELEGATOR(registry, Gemv<float>, DelegatorParam,
                                   MACE_HIP_DELEGATOR_KEY(Gemv, RT_CPU, float, kCpuImplType));
  if (st != MaceStatus::MACE_SUCCESS) return st;
  st = MACE_HIP_REGISTER_DELEGATOR(registry, Gemv<uint8_t>, DelegatorParam,
                                   MACE_HIP_DELEGATOR_KEY(Gemv, RT_CPU, uint8_t, kCpuImplType));
  if (st != MaceStatus::MACE_SUCCESS) return st;
  st = MACE_HIP_REGISTER_DELEGATOR(registry, Gemv<int32_t>, DelegatorParam,
                                   MACE_HIP_DELEGATOR_KEY(Gemv, RT_CPU, int32_t, kCpuImplType));
  if (st != MaceStatus::MACE_SUCCESS) return st;
  // The general key is the one Conv2dOp asks for on a host without NEON -- the only kind an
  // MI355X has (mace/ops/conv_2d.cc:88-91); the K1x1 tag serves a NEON build's request.
  st = MACE_HIP_REGISTER_DELEGATOR(registry, Conv2d<float>, delegator::Conv2dParam,
                                   MACE_HIP_DELEGATOR_KEY(Conv2d, RT_CPU, float, kCpuImplType));
  if (st != MaceStatus::MACE_SUCCESS) return st;
  return MACE_HIP_REGISTER_DELEGATOR(
      registry, Conv2dK1x1<float>, delegator::Conv2dParam,
      MACE_HIP_DELEGATOR_KEY_EX(Conv2d, RT_CPU, float, kCpuImplType, K1x1));
}

}  // namespace hip

// ---- ops: shape derivation and dispatch ------------------------------------------------------------------
namespace ops {

struct MatMulShape {
  index_t rows, cols, depth, batch;
  index_t lhs_rows, lhs_cols, rhs_rows, rhs_cols;
  bool lhs_batched, rhs_batched;
  std::vector<index_t> output_shape;
};

// MatMulOpBase::Validate (mace/ops/matmul.cc:55-83) + the head of Run (:117-154)
inline MaceStatus MatMulInferShape(const Tensor *A, const Tensor *B, bool transpose_a,
                                   bool transpose_b, MatMulShape *s) {
  const index_t lhs_rank = A->dim_size(), rhs_rank = B->dim_size();
  if (lhs_rank < 2 || rhs_rank < 2) return MaceStatus::MACE_INVALID_ARGS;
  if (lhs_rank == rhs_rank) {
    for (index_t i = 0; i < lhs_rank - 2; ++i)
      if (A->dim(i) != B->dim(i)) return MaceStatus::MACE_INVALID_ARGS;
  } else if (lhs_rank != 2 && rhs_rank != 2) {
    return MaceStatus::MACE_INVALID_ARGS;
  }
  s->lhs_rows = A->dim(lhs_rank - 2); s->lhs_cols = A->dim(lhs_rank - 1);
  s->rhs_rows = B->dim(rhs_rank - 2); s->rhs_cols = B->dim(rhs_rank - 1);
  const index_t lhs_depth = transpose_a ? s->lhs_rows : s->lhs_cols;
  const index_t rhs_depth = transpose_b ? s->rhs_cols : s->rhs_rows;
  if (lhs_depth != rhs_depth) return MaceStatus::MACE_INVALID_ARGS;
  s->rows = transpose_a ? s->lhs_cols : s->lhs_rows;
  s->cols = transpose_b ? s->rhs_rows : s->rhs_cols;
  s->depth = lhs_depth;
  auto lead = [](const Tensor *t) {
    return std::accumulate(t->shape().begin(), t->shape().end() - 2, index_t(1),
                           std::multiplies<index_t>());
  };
  if (lhs_rank >= rhs_rank) { s->output_shape = A->shape(); s->batch = lead(A); }
  else { s->output_shape = B->shape(); s->batch = lead(B); }
  s->output_shape[s->output_shape.size() - 2] = s->rows;
  s->output_shape[s->output_shape.size() - 1] = s->cols;
  s->lhs_batched = !(lhs_rank < rhs_rank);
  s->rhs_batched = !(rhs_rank < lhs_rank);
  return MaceStatus::MACE_SUCCESS;
}

// MatMulOp<RT_CPU, float>::Run (mace/ops/matmul.cc:110-215).  The optional bias of the Gemm
// branch (:195-211), a loop over the finished result in the reference, is added by the GEMM
// kernel as it stores the result (mace_hip_matmul_f32): one launch, host or device tensors.
class MatMulOpFloat {
 public:
  MatMulOpFloat(OpDelegatorRegistry *registry, bool transpose_a, bool transpose_b)
      : transpose_a_(transpose_a), transpose_b_(transpose_b) {
    auto gc = registry->GetCreator(MACE_HIP_DELEGATOR_KEY(Gemm, RT_CPU, float, kCpuImplType));
    auto vc = registry->GetCreator(MACE_HIP_DELEGATOR_KEY(Gemv, RT_CPU, float, kCpuImplType));
    if (gc) gemm_.reset(static_cast<delegator::Gemm *>(gc(delegator::GemmParam()).release()));
    if (vc) gemv_.reset(static_cast<delegator::Gemv *>(vc(DelegatorParam()).release()));
  }
  MaceStatus Run(OpContext *context, const Tensor *lhs, const Tensor *rhs, const Tensor *bias,
                 Tensor *C) {
    if (!gemm_ || !gemv_) return MaceStatus::MACE_RUNTIME_ERROR;
    MatMulShape s;
    MaceStatus st = MatMulInferShape(lhs, rhs, transpose_a_, transpose_b_, &s);
    if (st != MaceStatus::MACE_SUCCESS) return st;
    if ((st = C->Resize(s.output_shape)) != MaceStatus::MACE_SUCCESS) return st;
    if (s.rows == 1 && transpose_b_)
      return gemv_->Compute(context, rhs, lhs, bias, s.batch, s.cols, s.depth, s.rhs_batched,
                            s.lhs_batched, C);
    if (s.cols == 1 && !transpose_a_)
      return gemv_->Compute(context, lhs, rhs, bias, s.batch, s.rows, s.depth, s.lhs_batched,
                            s.rhs_batched, C);
    if (bias == nullptr)
      return gemm_->Compute(context, lhs, rhs, s.batch, s.lhs_rows, s.lhs_cols, s.rhs_rows,
                            s.rhs_cols, transpose_a_, transpose_b_, false, s.lhs_batched,
                            s.rhs_batched, C);
    // "bias' dim should be <= 2." (:196-197), checked before anything is written
    if (bias->dim_size() != 1 || bias->dim(0) != s.cols) return MaceStatus::MACE_INVALID_ARGS;
    if (!SamePlacement(C, {lhs, rhs, bias})) return MaceStatus::MACE_INVALID_ARGS;
    auto fn = C->on_device() ? mace_hip_matmul_f32 : mace_hip_matmul_f32_host;
    return ToStatus(fn(context->hip(), lhs->data<float>(), rhs->data<float>(), bias->data<float>(),
                       s.batch, s.lhs_rows, s.lhs_cols, s.rhs_rows, s.rhs_cols, transpose_a_,
                       transpose_b_, s.lhs_batched, s.rhs_batched, C->mutable_data<float>()));
  }

 private:
  bool transpose_a_, transpose_b_;
  std::unique_ptr<delegator::Gemm> gemm_;
  std::unique_ptr<delegator::Gemv> gemv_;
};

// MatMulOp<RT_CPU, uint8_t>::Run (mace/ops/matmul.cc:397-483) with MatMulFixpointImpl
// (:227-394): transposes become Col orders, the result is RowMajor, no bias; the uint8 result
// uses the pipeline MakeNoBias(A.scale, B.scale, C.scale, C.zero_point), the int32 result
// sets C.scale = A.scale * B.scale and C.zero_point = 0.  The gemmlowp call is not behind a
// delegator in the reference, so the op calls the C ABI directly.
// A constant operand (is_weight()) is kept resident across Run() calls (WeightRegistration).
class MatMulOpQuant {
 public:
  MatMulOpQuant(bool transpose_a, bool transpose_b, DataType output_type)
      : transpose_a_(transpose_a), transpose_b_(transpose_b), output_type_(output_type) {}
  MaceStatus Run(OpContext *context, const Tensor *A, const Tensor *B, Tensor *C) {
    MatMulShape s;
    MaceStatus st = MatMulInferShape(A, B, transpose_a_, transpose_b_, &s);
    if (st != MaceStatus::MACE_SUCCESS) return st;
    if ((st = C->Resize(s.output_shape)) != MaceStatus::MACE_SUCCESS) return st;
    if (!SamePlacement(C, {A, B})) return MaceStatus::MACE_INVALID_ARGS;
    const int a_order = transpose_a_ ? MACE_HIP_COL_MAJOR : MACE_HIP_ROW_MAJOR;
    const int b_order = transpose_b_ ? MACE_HIP_COL_MAJOR : MACE_HIP_ROW_MAJOR;
    weight_a_.Note(context, A, static_cast<size_t>(A->size()));
    weight_b_.Note(context, B, static_cast<size_t>(B->size()));
    if (output_type_ == DT_INT32) {
      C->SetScale(A->scale() * B->scale());
      C->SetZeroPoint(0);
      auto fn = C->on_device() ? mace_hip_gemm_q8_i32 : mace_hip_gemm_q8_i32_host;
      return ToStatus(fn(context->hip(), A->data<uint8_t>(), a_order, B->data<uint8_t>(),
                         b_order, C->mutable_data<int32_t>(), MACE_HIP_ROW_MAJOR, s.batch,
                         s.rows, s.depth, s.cols, s.lhs_batched, s.rhs_batched,
                         -A->zero_point(), -B->zero_point()));
    }
    int32_t multiplier = 0;
    int shift = 0;
    if (mace_hip_get_output_multiplier_and_shift(A->scale(), B->scale(), C->scale(),
                                                 &multiplier, &shift) != MACE_HIP_SUCCESS)
      return MaceStatus::MACE_INVALID_ARGS;
    auto fn = C->on_device() ? mace_hip_gemm_q8_u8 : mace_hip_gemm_q8_u8_host;
    return ToStatus(fn(context->hip(), A->data<uint8_t>(), a_order, B->data<uint8_t>(), b_order,
                       C->mutable_data<uint8_t>(), MACE_HIP_ROW_MAJOR, s.batch, s.rows,
                       s.depth, s.cols, s.lhs_batched, s.rhs_batched, -A->zero_point(),
                       -B->zero_point(), nullptr, multiplier, shift, C->zero_point(), 0, 255));
  }

 private:
  bool transpose_a_, transpose_b_;
  DataType output_type_;
  WeightRegistration weight_a_, weight_b_;
};

// FullyConnectedOp<RT_CPU, uint8_t>::Run (mace/ops/fully_connected.cc:141-179) and the float op
// (:82-121): weight OIHW, output {N,1,1,O} (uint8) / {N,O,1,1} (float).  The float op runs its
// Activation delegator on the Gemv's output (:62-75,121: the op's "activation" / "max_limit"
// arguments; mace/ops/ref/activation.cc:61-75); the quantized op has none (the converter folds a
// quantized ReLU into the output range).  With the GPU Gemv the activation is applied as the sums
// are stored; with any other Gemv delegator it is the reference's host loop.  NOOP, RELU and RELUX
// are applied; any other type makes Run return MACE_UNSUPPORTED before anything is computed.
template <typename T>
class FullyConnectedOp {
 public:
  explicit FullyConnectedOp(OpDelegatorRegistry *registry, ActivationType activation = NOOP,
                            float max_limit = 0.f)
      : activation_(activation), max_limit_(max_limit) {
    auto vc = registry->GetCreator(MACE_HIP_DELEGATOR_KEY(Gemv, RT_CPU, T, kCpuImplType));
    if (vc) gemv_.reset(static_cast<delegator::Gemv *>(vc(DelegatorParam()).release()));
  }
  MaceStatus Run(OpContext *context, const Tensor *input, const Tensor *weight,
                 const Tensor *bias, Tensor *output) {
    if (!gemv_) return MaceStatus::MACE_RUNTIME_ERROR;
    if (input->dim_size() != 4 || weight->dim_size() != 4 || input->dim(1) != weight->dim(1) ||
        input->dim(2) != weight->dim(2) || input->dim(3) != weight->dim(3))
      return MaceStatus::MACE_INVALID_ARGS;
    if (bias && weight->dim(0) != bias->dim(0)) return MaceStatus::MACE_INVALID_ARGS;
    std::vector<index_t> out_shape =
        std::is_same<T, uint8_t>::value
            ? std::vector<index_t>{input->dim(0), 1, 1, weight->dim(0)}
            : std::vector<index_t>{input->dim(0), weight->dim(0), 1, 1};
    MaceStatus st = output->Resize(out_shape);
    if (st != MaceStatus::MACE_SUCCESS) return st;
    const index_t input_size = weight->dim(1) * weight->dim(2) * weight->dim(3);
    if (std::is_same<T, float>::value) {
      if (activation_ != NOOP && activation_ != RELU && activation_ != RELUX)
        return MaceStatus::MACE_UNSUPPORTED;
      if (auto *fused = dynamic_cast<hip::Gemv<float> *>(gemv_.get()))
        return fused->ComputeFused(context, weight, input, bias, input->dim(0), weight->dim(0),
                                   input_size, false, true, activation_, max_limit_, output);
    }
    st = gemv_->Compute(context, weight, input, bias, input->dim(0), weight->dim(0), input_size,
                        false, true, output);
    if (st != MaceStatus::MACE_SUCCESS || !std::is_same<T, float>::value || activation_ == NOOP)
      return st;
    if (output->on_device()) return MaceStatus::MACE_UNSUPPORTED;   // host loop below
    float *o = output->template mutable_data<float>();
    for (index_t i = 0; i < output->size(); ++i)
      o[i] = std::max(0.f, activation_ == RELUX ? std::min(max_limit_, o[i]) : o[i]);
    return st;
  }

 private:
  ActivationType activation_;
  float max_limit_;
  std::unique_ptr<delegator::Gemv> gemv_;
};

using ::mace_hip::Padding;
using ::mace_hip::VALID;
using ::mace_hip::SAME;
using ::mace_hip::FULL;

// Conv2dOp<RT_CPU, uint8_t>::Run (mace/ops/conv_2d.cc:201-318): NHWC input, OHWI filter, NHWC
// output, dilation 1.  The output shape comes from the padding type (CalcPaddingAndOutputSize)
// or, when explicit paddings are given, from the FLOOR rule (CalcOutputSize), exactly as the
// op does (:213-235).  A fused quantized ReLUx is the clamp range.
class Conv2dOpQuant {
 public:
  Conv2dOpQuant(std::vector<int> strides = {1, 1}, Padding padding_type = SAME,
                std::vector<int> paddings = {}, std::vector<int> dilations = {1, 1},
                int clamp_min = 0, int clamp_max = 255)
      : strides_(std::move(strides)), padding_type_(padding_type), paddings_(std::move(paddings)),
        dilations_(std::move(dilations)), clamp_min_(clamp_min), clamp_max_(clamp_max) {}
  MaceStatus Run(OpContext *context, const Tensor *input, const Tensor *filter,
                 const Tensor *bias, Tensor *output) {
    if (input->dim_size() != 4 || filter->dim_size() != 4) return MaceStatus::MACE_INVALID_ARGS;
    if (strides_.size() != 2 || dilations_.size() != 2) return MaceStatus::MACE_INVALID_ARGS;
    // "Quantization convolution does not support dilation > 1 yet." (:207-208)
    if (dilations_[0] != 1 || dilations_[1] != 1) return MaceStatus::MACE_INVALID_ARGS;
    if (filter->dim(3) != input->dim(3)) return MaceStatus::MACE_INVALID_ARGS;
    if (bias && bias->dim(0) != filter->dim(0)) return MaceStatus::MACE_INVALID_ARGS;
    int64_t out_h = 0, out_w = 0;
    int pads[2] = {0, 0};
    if (paddings_.empty()) {
      MaceStatus st = ToStatus(mace_hip_calc_padding_and_output_size(
          input->dim(1), input->dim(2), filter->dim(1), filter->dim(2), dilations_[0],
          dilations_[1], strides_[0], strides_[1], padding_type_, &out_h, &out_w, &pads[0],
          &pads[1]));
      if (st != MaceStatus::MACE_SUCCESS) return st;
    } else {
      if (paddings_.size() != 2 || strides_[0] <= 0 || strides_[1] <= 0)
        return MaceStatus::MACE_INVALID_ARGS;
      pads[0] = paddings_[0];
      pads[1] = paddings_[1];
      out_h = static_cast<int64_t>(
          std::floor(1.0 * (input->dim(1) + pads[0] - filter->dim(1)) / strides_[0]) + 1);
      out_w = static_cast<int64_t>(
          std::floor(1.0 * (input->dim(2) + pads[1] - filter->dim(2)) / strides_[1]) + 1);
    }
    if (!SamePlacement(output, {input, filter, bias})) return MaceStatus::MACE_INVALID_ARGS;
    MaceStatus st = output->Resize({input->dim(0), out_h, out_w, filter->dim(0)});
    if (st != MaceStatus::MACE_SUCCESS) return st;
    weight_.Note(context, filter, static_cast<size_t>(filter->size()));   // filters are constants
    if (bias) bias_.Note(context, bias, sizeof(int32_t) * static_cast<size_t>(bias->size()));
    auto fn = output->on_device() ? mace_hip_conv2d_q8_nhwc : mace_hip_conv2d_q8_nhwc_host;
    return ToStatus(fn(context->hip(), input->data<uint8_t>(), filter->data<uint8_t>(),
                       bias ? bias->data<int32_t>() : nullptr, input->dim(0), input->dim(1),
                       input->dim(2), input->dim(3), filter->dim(0), filter->dim(1),
                       filter->dim(2), strides_[0], strides_[1], pads[0], pads[1], input->scale(),
                       input->zero_point(), filter->scale(), filter->zero_point(),
                       bias ? bias->scale() : 0.f, output->scale(), output->zero_point(),
                       clamp_min_, clamp_max_, output->mutable_data<uint8_t>()));
  }

 private:
  std::vector<int> strides_;
  Padding padding_type_;
  std::vector<int> paddings_, dilations_;
  int clamp_min_, clamp_max_;
  WeightRegistration weight_, bias_;
};

// The 1x1 / stride 1 / no padding case under its earlier name.
class Conv2dK1x1OpQuant {
 public:
  Conv2dK1x1OpQuant(int clamp_min = 0, int clamp_max = 255)
      : op_({1, 1}, VALID, {}, {1, 1}, clamp_min, clamp_max) {}
  MaceStatus Run(OpContext *context, const Tensor *input, const Tensor *filter,
                 const Tensor *bias, Tensor *output) {
    if (filter->dim_size() == 4 && (filter->dim(1) != 1 || filter->dim(2) != 1))
      return MaceStatus::MACE_UNSUPPORTED;
    return op_.Run(context, input, filter, bias, output);
  }

 private:
  Conv2dOpQuant op_;
};

// Conv2dOp<RT_CPU, float>::Run (mace/ops/conv_2d.cc:82-173): picks the delegator key on the first
// run -- the general key, or on a NEON build the tag of the filter geometry (only the K1x1 tag
// is mirrored) -- creates the delegator through the registry, runs it, then BiasAdd and
// Activation (ref/bias_add.cc:74-100 NCHW, ref/activation.cc:61-75 NOOP / RELU / RELUX).  With the
// GPU delegator the last two are applied as the result is stored; with any other delegator they
// are the reference's host loops.
class Conv2dOpFloat {
 public:
  Conv2dOpFloat(OpDelegatorRegistry *registry, std::vector<int> strides = {1, 1},
                Padding padding_type = SAME, std::vector<int> paddings = {},
                std::vector<int> dilations = {1, 1}, ActivationType activation = NOOP,
                float max_limit = 0.f, ImplType impl = kCpuImplType)
      : registry_(registry), strides_(std::move(strides)), padding_type_(padding_type),
        paddings_(std::move(paddings)), dilations_(std::move(dilations)), activation_(activation),
        max_limit_(max_limit), impl_(impl) {}
  MaceStatus Run(OpContext *context, const Tensor *input, const Tensor *filter,
                 const Tensor *bias, Tensor *output) {
    if (input->dim_size() != 4 || filter->dim_size() != 4 || strides_.size() != 2 ||
        dilations_.size() != 2)
      return MaceStatus::MACE_INVALID_ARGS;
    if (!conv_) {
      DelegatorInfo tag = MACE_HIP_DELEGATOR_KEY(Conv2d, RT_CPU, float, impl_);
      if (impl_ == NEON && filter->dim(2) == 1 && filter->dim(3) == 1 && strides_[0] == 1 &&
          strides_[1] == 1 && dilations_[0] == 1 && dilations_[1] == 1)
        tag = MACE_HIP_DELEGATOR_KEY_EX(Conv2d, RT_CPU, float, impl_, K1x1);
      DelegatorCreator creator = registry_->GetCreator(tag);
      if (!creator) return MaceStatus::MACE_RUNTIME_ERROR;   // LOG(FATAL) in the reference
      delegator::Conv2dParam param(strides_, dilations_, paddings_, padding_type_);
      conv_.reset(static_cast<delegator::Conv2d *>(creator(param).release()));
    }
    if (auto *fused = dynamic_cast<hip::Conv2d<float> *>(conv_.get()))
      return fused->ComputeFused(context, input, filter, bias, activation_, max_limit_, output);
    MaceStatus st = conv_->Compute(context, input, filter, output);
    if (st != MaceStatus::MACE_SUCCESS) return st;
    if (output->on_device()) return MaceStatus::MACE_UNSUPPORTED;   // host loops below
    float *o = output->mutable_data<float>();
    const index_t n = output->dim(0), c = output->dim(1), hw = output->dim(2) * output->dim(3);
    for (index_t i = 0; i < n * c; ++i)
      for (index_t p = 0; p < hw; ++p) {
        float v = o[i * hw + p];
        if (bias) v += bias->data<float>()[i % c];
        if (activation_ == RELU) v = std::max(0.f, v);
        if (activation_ == RELUX) v = std::max(0.f, std::min(max_limit_, v));
        o[i * hw + p] = v;
      }
    return st;
  }

 private:
  OpDelegatorRegistry *registry_;
  std::vector<int> strides_;
  Padding padding_type_;
  std::vector<int> paddings_, dilations_;
  ActivationType activation_;
  float max_limit_;
  ImplType impl_;
  std::unique_ptr<delegator::Conv2d> conv_;
};

// arm::Conv2dK3x3Winograd<float>::Compute (mace/ops/arm/base/conv_2d_3x3_winograd.cc:31-236): a
// caller of delegator::Gemm.  3x3 filter, stride 1, NCHW.  Output tiles of 2x2 (6x6 when the
// input is larger than 16x16, :43-46); the input is zero-padded so that whole tiles cover the
// (padded) output, every (tile + 2)^2 patch is transformed (B^T d B), the filter likewise
// (G g G^T), and the products over the input channels are ONE batched Gemm per image --
// batch = (tile + 2)^2, lhs = transformed filter [area][cout][cin], rhs = transformed input
// [area][cin][tiles], both batched, row-major (:191-204) -- followed by the output transform
// (A^T m A).  The transforms are host loops written from the standard matrices of the
// algorithm (the reference has NEON code for the same matrices); the Gemm is the delegator's.
// Host tensors only: the transforms read and write the tensors' memory directly.
class Conv2dK3x3WinogradOp {
 public:
  Conv2dK3x3WinogradOp(OpDelegatorRegistry *registry, Padding padding_type = SAME,
                       std::vector<int> paddings = {})
      : padding_type_(padding_type), paddings_(std::move(paddings)) {
    auto gc = registry->GetCreator(MACE_HIP_DELEGATOR_KEY(Gemm, RT_CPU, float, kCpuImplType));
    if (gc) gemm_.reset(static_cast<delegator::Gemm *>(gc(delegator::GemmParam()).release()));
  }
  MaceStatus Run(OpContext *context, const Tensor *input, const Tensor *filter, Tensor *output) {
    if (!gemm_) return MaceStatus::MACE_RUNTIME_ERROR;
    if (input->dim_size() != 4 || filter->dim_size() != 4 || filter->dim(2) != 3 ||
        filter->dim(3) != 3 || filter->dim(1) != input->dim(1) || input->on_device())
      return MaceStatus::MACE_INVALID_ARGS;
    const index_t batch = input->dim(0), cin = input->dim(1), in_h = input->dim(2),
                  in_w = input->dim(3), cout = filter->dim(0);
    const int t = (in_h > 16 && in_w > 16) ? 6 : 2;   // output tile
    const int a = t + 2, area = a * a;                 // input tile and its area
    int64_t out_h = 0, out_w = 0;
    int pads[2] = {0, 0};
    if (paddings_.empty()) {
      MaceStatus st = ToStatus(mace_hip_calc_padding_and_output_size(
          in_h, in_w, 3, 3, 1, 1, 1, 1, padding_type_, &out_h, &out_w, &pads[0], &pads[1]));
      if (st != MaceStatus::MACE_SUCCESS) return st;
    } else {
      if (paddings_.size() != 2) return MaceStatus::MACE_INVALID_ARGS;
      pads[0] = paddings_[0]; pads[1] = paddings_[1];
      out_h = in_h + pads[0] - 2; out_w = in_w + pads[1] - 2;
    }
    if (out_h <= 0 || out_w <= 0) return MaceStatus::MACE_INVALID_ARGS;
    MaceStatus st = output->Resize({batch, cout, out_h, out_w});
    if (st != MaceStatus::MACE_SUCCESS) return st;
    // arm/base/conv_2d.cc:97-119: output rounded up to whole tiles, input padded to match
    const index_t poh = (out_h + t - 1) / t * t, pow_ = (out_w + t - 1) / t * t;
    const index_t pih = std::max<index_t>(in_h + pads[0], poh + 2);
    const index_t piw = std::max<index_t>(in_w + pads[1], pow_ + 2);
    const int top = pads[0] >> 1, left = pads[1] >> 1;
    const index_t th = poh / t, tw = pow_ / t, tiles = th * tw;
    const float *BT = t == 2 ? kBT4 : kBT8, *G = t == 2 ? kG4 : kG8, *AT = t == 2 ? kAT4 : kAT8;

    // filter [cout][cin][3][3] -> U [area][cout][cin] = G g G^T.  As in the reference, the
    // transformed filter of a constant filter is computed once and kept (conv_2d_3x3_winograd.cc:
    // 120-143: redone only when the filter is not a weight or the tile size changes); it is the
    // constant left-hand side of every Gemm call below, so it also stays on the GPU.
    std::vector<float> V((size_t)area * cin * tiles), M((size_t)area * cout * tiles), tmp(a * 3), d(area),
        w(area);
    const float *f = filter->data<float>();
    const bool keep = filter->is_weight() && t == u_tile_ && f == u_filter_ &&
                      U_.size() == (size_t)area * cout * cin;
    if (!keep) {
      u_resident_.Release();
      U_.assign((size_t)area * cout * cin, 0.f);
      for (index_t oc = 0; oc < cout; ++oc)
        for (index_t ic = 0; ic < cin; ++ic) {
          const float *g = f + (oc * cin + ic) * 9;
          for (int i = 0; i < a; ++i)
            for (int j = 0; j < 3; ++j)
              tmp[i * 3 + j] = G[i * 3] * g[j] + G[i * 3 + 1] * g[3 + j] + G[i * 3 + 2] * g[6 + j];
          for (int i = 0; i < a; ++i)
            for (int j = 0; j < a; ++j)
              U_[((size_t)(i * a + j) * cout + oc) * cin + ic] =
                  tmp[i * 3] * G[j * 3] + tmp[i * 3 + 1] * G[j * 3 + 1] + tmp[i * 3 + 2] * G[j * 3 + 2];
        }
      u_tile_ = t;
      u_filter_ = f;
    }
    Tensor Ut(U_.data(), DT_FLOAT, {area, cout, cin}, 0.f, 0, /*is_weight=*/filter->is_weight()),
        Vt(V.data(), DT_FLOAT, {area, cin, tiles}), Mt(M.data(), DT_FLOAT, {area, cout, tiles});
    u_resident_.Note(context, &Ut, sizeof(float) * U_.size());
    const float *x = input->data<float>();
    float *y = output->mutable_data<float>();
    for (index_t b = 0; b < batch; ++b) {
      // input patches -> V [area][cin][tiles] = B^T d B (zero outside the image)
      for (index_t ic = 0; ic < cin; ++ic)
        for (index_t ty = 0; ty < th; ++ty)
          for (index_t tx = 0; tx < tw; ++tx) {
            for (int i = 0; i < a; ++i)
              for (int j = 0; j < a; ++j) {
                const index_t py = ty * t + i, px = tx * t + j;   // in the padded image
                const index_t iy = py - top, ix = px - left;
                const bool in = py < pih && px < piw && iy >= 0 && iy < in_h && ix >= 0 && ix < in_w;
                d[i * a + j] = in ? x[((b * cin + ic) * in_h + iy) * in_w + ix] : 0.f;
              }
            Sandwich(BT, d.data(), a, a, w.data());
            for (int k = 0; k < area; ++k)
              V[((size_t)k * cin + ic) * tiles + ty * tw + tx] = w[k];
          }
      // conv_2d_3x3_winograd.cc:191-204
      st = gemm_->Compute(context, &Ut, &Vt, area, cout, cin, cin, tiles, false, false, false, true,
                          true, &Mt);
      if (st != MaceStatus::MACE_SUCCESS) return st;
      // M [area][cout][tiles] -> output tiles = A^T m A, cropped to the output
      for (index_t oc = 0; oc < cout; ++oc)
        for (index_t ty = 0; ty < th; ++ty)
          for (index_t tx = 0; tx < tw; ++tx) {
            for (int k = 0; k < area; ++k) d[k] = M[((size_t)k * cout + oc) * tiles + ty * tw + tx];
            Sandwich(AT, d.data(), t, a, w.data());
            for (int i = 0; i < t; ++i)
              for (int j = 0; j < t; ++j) {
                const index_t oy = ty * t + i, ox = tx * t + j;
                if (oy < out_h && ox < out_w)
                  y[((b * cout + oc) * out_h + oy) * out_w + ox] = w[i * t + j];
              }
          }
    }
    return MaceStatus::MACE_SUCCESS;
  }

 private:
  // out (r x r) = L (r x a) * m (a x a) * L^T
  static void Sandwich(const float *L, const float *m, int r, int a, float *out) {
    float tmp[64];
    for (int i = 0; i < r; ++i)
      for (int j = 0; j < a; ++j) {
        float s = 0.f;
        for (int k = 0; k < a; ++k) s += L[i * a + k] * m[k * a + j];
        tmp[i * a + j] = s;
      }
    for (int i = 0; i < r; ++i)
      for (int j = 0; j < r; ++j) {
        float s = 0.f;
        for (int k = 0; k < a; ++k) s += tmp[i * a + k] * L[j * a + k];
        out[i * r + j] = s;
      }
  }
  // F(2x2, 3x3) and F(6x6, 3x3): interpolation points 0, +-1 (and +-2, +-1/2), infinity
  static constexpr float kBT4[16] = {1, 0, -1, 0, 0, 1, 1, 0, 0, -1, 1, 0, 0, 1, 0, -1};
  static constexpr float kG4[12] = {1, 0, 0, .5f, .5f, .5f, .5f, -.5f, .5f, 0, 0, 1};
  static constexpr float kAT4[8] = {1, 1, 1, 0, 0, 1, -1, -1};
  static constexpr float kBT8[64] = {
      1, 0, -5.25f, 0, 5.25f, 0, -1, 0,       0, 1, 1, -4.25f, -4.25f, 1, 1, 0,
      0, -1, 1, 4.25f, -4.25f, -1, 1, 0,      0, .5f, .25f, -2.5f, -1.25f, 2, 1, 0,
      0, -.5f, .25f, 2.5f, -1.25f, -2, 1, 0,  0, 2, 4, -2.5f, -5, .5f, 1, 0,
      0, -2, 4, 2.5f, -5, -.5f, 1, 0,         0, -1, 0, 5.25f, 0, -5.25f, 0, 1};
  static constexpr float kG8[24] = {
      1, 0, 0,  -2.f / 9, -2.f / 9, -2.f / 9,  -2.f / 9, 2.f / 9, -2.f / 9,
      1.f / 90, 1.f / 45, 2.f / 45,  1.f / 90, -1.f / 45, 2.f / 45,
      32.f / 45, 16.f / 45, 8.f / 45,  32.f / 45, -16.f / 45, 8.f / 45,  0, 0, 1};
  static constexpr float kAT8[48] = {
      1, 1, 1, 1, 1, 1, 1, 0,               0, 1, -1, 2, -2, .5f, -.5f, 0,
      0, 1, 1, 4, 4, .25f, .25f, 0,         0, 1, -1, 8, -8, .125f, -.125f, 0,
      0, 1, 1, 16, 16, .0625f, .0625f, 0,   0, 1, -1, 32, -32, .03125f, -.03125f, 1};
  Padding padding_type_;
  std::vector<int> paddings_;
  std::unique_ptr<delegator::Gemm> gemm_;
  std::vector<float> U_;              // transformed filter, kept while the filter is a constant
  int u_tile_ = 0;
  const float *u_filter_ = nullptr;
  WeightRegistration u_resident_;
};

// DynamicLSTMOp<RT_CPU, float>::Run (mace/ops/dynamic_lstm.cc:160-372), a caller of
// delegator::Gemv: per batch and output frame, affine a (weights_a [a_out][input_dim +
// prev_out_dim] against the input frame appended with the delayed output, :296-310), the LSTM
// nonlinearity with peephole parameters (mace/ops/common/lstm.h:29-84), the cell scaled
// (:83-104), affine b (weights_b [out_dim][cell_dim], :328-337), and the delayed output / cell
// ring buffers and caches (:339-366).  Both affines are batch-1 Gemv calls with nothing batched
// and an optional bias; everything else is the reference's host code restated.
struct DynamicLSTMArgs {
  int prev_out_delay = 0, prev_cell_delay = 0, prev_out_offset = 0, prev_out_dim = 0,
      prev_cell_dim = 0, subsample_factor = 1;
  float scale = 1.0f;
  std::vector<index_t> forward_indexes, cell_cache_indexes, out_cache_indexes;
};
class DynamicLSTMOp {
 public:
  DynamicLSTMOp(OpDelegatorRegistry *registry, DynamicLSTMArgs args) : a_(std::move(args)) {
    auto vc = registry->GetCreator(MACE_HIP_DELEGATOR_KEY(Gemv, RT_CPU, float, kCpuImplType));
    if (vc) gemv_.reset(static_cast<delegator::Gemv *>(vc(DelegatorParam()).release()));
  }
  MaceStatus Run(OpContext *context, const Tensor *input, const Tensor *prev_out,
                 const Tensor *prev_cell, const Tensor *weights_a, const Tensor *lstm_params,
                 const Tensor *weights_b, const Tensor *bias_a, const Tensor *bias_b,
                 Tensor *output, Tensor *out_cache, Tensor *cell_cache) {
    if (!gemv_) return MaceStatus::MACE_RUNTIME_ERROR;
    const index_t rank = input->dim_size();
    // Validate (:81-118)
    if (rank < 2 || a_.prev_cell_delay >= 0 || a_.prev_out_delay >= 0 || a_.subsample_factor <= 0 ||
        a_.prev_cell_delay % a_.subsample_factor != 0 || a_.prev_out_delay % a_.subsample_factor != 0 ||
        a_.prev_out_dim <= 0 || a_.prev_cell_dim <= 0)
      return MaceStatus::MACE_INVALID_ARGS;
    const index_t chunk = input->dim(rank - 2), input_dim = input->dim(rank - 1);
    for (index_t fi : a_.forward_indexes)
      if (fi < 0 || fi >= chunk) return MaceStatus::MACE_INVALID_ARGS;
    const index_t batch = std::accumulate(input->shape().begin(), input->shape().end() - 2,
                                          index_t(1), std::multiplies<index_t>());
    const index_t a_in = input_dim + a_.prev_out_dim, a_out = weights_a->dim(0);
    if (a_in != weights_a->dim(1)) return MaceStatus::MACE_INVALID_ARGS;
    const index_t lstm_in = a_out + a_.prev_cell_dim, cell_dim = lstm_in / 5;
    if (lstm_in != cell_dim * 5 || lstm_params->dim(0) != 3 || lstm_params->dim(1) != cell_dim ||
        cell_dim != a_.prev_cell_dim)
      return MaceStatus::MACE_INVALID_ARGS;
    const index_t out_dim = weights_b->dim(0);
    if (weights_b->dim(1) != cell_dim || a_.prev_out_offset + a_.prev_out_dim > out_dim)
      return MaceStatus::MACE_INVALID_ARGS;
    const index_t out_buf_chunk = std::abs(a_.prev_out_delay / a_.subsample_factor);
    const index_t cell_buf_chunk = std::abs(a_.prev_cell_delay / a_.subsample_factor);
    const index_t out_chunk = (index_t)a_.forward_indexes.size();

    std::vector<index_t> shape = input->shape();
    shape[rank - 1] = out_dim;   // (the reference keeps the input's chunk here, :264-266)
    MaceStatus st = output->Resize(shape);
    shape[rank - 1] = a_.prev_out_dim; shape[rank - 2] = out_buf_chunk;
    if (st == MaceStatus::MACE_SUCCESS) st = out_cache->Resize(shape);
    shape[rank - 1] = a_.prev_cell_dim; shape[rank - 2] = cell_buf_chunk;
    if (st == MaceStatus::MACE_SUCCESS) st = cell_cache->Resize(shape);
    if (st != MaceStatus::MACE_SUCCESS) return st;

    std::vector<float> out_buf(out_buf_chunk * a_.prev_out_dim), cell_buf(cell_buf_chunk * cell_dim),
        va_in(a_in), va_out(a_out), vb_in(cell_dim), vb_out(out_dim);
    Tensor a_in_t(va_in.data(), DT_FLOAT, {1, a_in}), a_out_t(va_out.data(), DT_FLOAT, {1, a_out}),
        b_in_t(vb_in.data(), DT_FLOAT, {1, cell_dim}), b_out_t(vb_out.data(), DT_FLOAT, {1, out_dim});
    const float *x = input->data<float>(), *params = lstm_params->data<float>();
    float *y = output->mutable_data<float>();
    const bool unit_scale = std::abs(a_.scale - 1.f) < 1e-6;
    for (index_t b = 0; b < batch; ++b) {
      std::copy_n(prev_out->data<float>() + b * out_buf_chunk * a_.prev_out_dim, out_buf.size(),
                  out_buf.begin());
      std::copy_n(prev_cell->data<float>() + b * cell_buf_chunk * cell_dim, cell_buf.size(),
                  cell_buf.begin());
      for (index_t i = 0; i < out_chunk; ++i) {
        std::copy_n(x + (b * chunk + a_.forward_indexes[i]) * input_dim, input_dim, va_in.begin());
        std::copy_n(out_buf.data() + i % out_buf_chunk * a_.prev_out_dim, a_.prev_out_dim,
                    va_in.begin() + input_dim);
        st = gemv_->Compute(context, weights_a, &a_in_t, bias_a, 1, a_out, a_in, false, false, &a_out_t);
        if (st != MaceStatus::MACE_SUCCESS) return st;
        float *cell = cell_buf.data() + i % cell_buf_chunk * cell_dim;
        for (index_t c = 0; c < cell_dim; ++c) {   // common/lstm.h:64-81, embed_scales = false
          const float i_part = va_out[c], f_part = va_out[c + cell_dim],
                      c_part = va_out[c + 2 * cell_dim], o_part = va_out[c + 3 * cell_dim];
          const float c_prev = cell[c];
          const float i_t = Sigmoid(i_part + params[c] * c_prev);
          const float f_t = Sigmoid(f_part + params[c + cell_dim] * c_prev);
          const float c_t = f_t * 1.0f * c_prev + i_t * 1.0f * std::tanh(c_part);
          const float o_t = Sigmoid(o_part + params[c + 2 * cell_dim] * c_t);
          cell[c] = c_t;
          vb_in[c] = o_t * 1.0f * std::tanh(c_t);
        }
        if (!unit_scale)
          for (index_t c = 0; c < cell_dim; ++c) cell[c] *= a_.scale;
        st = gemv_->Compute(context, weights_b, &b_in_t, bias_b, 1, out_dim, cell_dim, false, false, &b_out_t);
        if (st != MaceStatus::MACE_SUCCESS) return st;
        std::copy_n(vb_out.begin(), out_dim, y + (b * out_chunk + i) * out_dim);
        float *cur_out = out_buf.data() + i % out_buf_chunk * a_.prev_out_dim;
        for (index_t k = 0; k < a_.prev_out_dim; ++k)
          cur_out[k] = unit_scale ? vb_out[a_.prev_out_offset + k] : vb_out[a_.prev_out_offset + k] * a_.scale;
        for (size_t k = 0; k < a_.out_cache_indexes.size(); ++k)
          if (i == a_.out_cache_indexes[k])
            std::copy_n(cur_out, a_.prev_out_dim,
                        out_cache->mutable_data<float>() + (b * out_buf_chunk + k) * a_.prev_out_dim);
        for (size_t k = 0; k < a_.cell_cache_indexes.size(); ++k)
          if (i == a_.cell_cache_indexes[k])
            std::copy_n(cell, cell_dim,
                        cell_cache->mutable_data<float>() + (b * cell_buf_chunk + k) * cell_dim);
      }
    }
    return MaceStatus::MACE_SUCCESS;
  }

 private:
  static float Sigmoid(float in) {   // mace/utils/math.h:63-70 ScalarSigmoid
    if (in > 0) return 1 / (1 + std::exp(-in));
    const float x = std::exp(in);
    return x / (x + 1.f);
  }
  DynamicLSTMArgs a_;
  std::unique_ptr<delegator::Gemv> gemv_;
};

// QuantizeOp<RT_CPU, uint8_t> (mace/ops/arm/q8/quantize.cc:31-72): float -> uint8.  An output
// tensor that already carries a scale is quantized with it; otherwise (or with
// find_range_every_time) the range is taken from the data and the scale / zero point found are
// stored on the output tensor.
class QuantizeOp {
 public:
  explicit QuantizeOp(bool non_zero = false, bool find_range_every_time = false)
      : non_zero_(non_zero), find_range_every_time_(find_range_every_time) {}
  MaceStatus Run(OpContext *context, const Tensor *input, Tensor *output) {
    if (!SamePlacement(output, {input})) return MaceStatus::MACE_INVALID_ARGS;
    MaceStatus st = output->Resize(input->shape());   // ResizeLike
    if (st != MaceStatus::MACE_SUCCESS) return st;
    if (!find_range_every_time_ && output->scale() > 0.f) {
      auto fn = output->on_device() ? mace_hip_quantize_tensor_u8 : mace_hip_quantize_tensor_u8_host;
      return ToStatus(fn(context->hip(), input->data<float>(), input->size(), output->scale(),
                         output->zero_point(), output->mutable_data<uint8_t>()));
    }
    float scale = 0.f;
    int32_t zero_point = 0;
    auto fn = output->on_device() ? mace_hip_quantize_tensor_dynamic_u8
                                  : mace_hip_quantize_tensor_dynamic_u8_host;
    st = ToStatus(fn(context->hip(), input->data<float>(), input->size(), non_zero_ ? 1 : 0,
                     output->mutable_data<uint8_t>(), &scale, &zero_point));
    if (st != MaceStatus::MACE_SUCCESS) return st;
    output->SetScale(scale);
    output->SetZeroPoint(zero_point);
    return st;
  }

 private:
  bool non_zero_, find_range_every_time_;
};

// DequantizeOp<RT_CPU, T> (mace/ops/arm/q8/quantize.cc:74-103), T = uint8_t or int32_t.
template <typename T>
class DequantizeOp {
 public:
  MaceStatus Run(OpContext *context, const Tensor *input, Tensor *output) {
    if (!SamePlacement(output, {input})) return MaceStatus::MACE_INVALID_ARGS;
    MaceStatus st = output->Resize(input->shape());
    if (st != MaceStatus::MACE_SUCCESS) return st;
    return ToStatus(Call(context->hip(), input->data<T>(), input->size(), input->scale(),
                         input->zero_point(), output->mutable_data<float>(), output->on_device()));
  }

 private:
  static int Call(mace_hip_ctx *c, const uint8_t *in, index_t n, float s, int32_t z, float *out,
                  bool dev) {
    return dev ? mace_hip_dequantize_tensor_u8(c, in, n, s, z, out)
               : mace_hip_dequantize_tensor_u8_host(c, in, n, s, z, out);
  }
  static int Call(mace_hip_ctx *c, const int32_t *in, index_t n, float s, int32_t z, float *out,
                  bool dev) {
    return dev ? mace_hip_dequantize_tensor_i32(c, in, n, s, z, out)
               : mace_hip_dequantize_tensor_i32_host(c, in, n, s, z, out);
  }
};

}  // namespace ops
}  // namespace mace_hip

#endif  // MACE_HIP_DELEGATOR_H_
