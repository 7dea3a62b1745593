// hyle_hip_compute.hpp -- C++17 host-side mirror, over the C ABI of hyle_hip.h, of the slice of
// `hyle::compute` a caller of the tensor hot path touches.  Names, argument meaning and error
// behaviour follow the reference so that code written against it reads the same:
//
//   auto context  = Context::create(hip::device(0)).value();                // include/hyle/compute/device.h:124-140
//   auto queue    = context.create_queue().value();                         // ...device.h:179-224
//   auto prepared = prepare(context, Binary{BinaryKind::kAdd}, a, b);       // include/hyle/compute/prepared_operation.h:313-317
//   auto run      = prepared->create_invocation().value();                  // ...prepared_operation.h:144-291
//   run.submit(queue, left_view, right_view, output)->wait();               // include/hyle/compute/completion.h:40
//
// Status / Result follow include/hyle/error/status.h and result.h (Result is std::expected in
// the reference; a small stand-in here because this toolchain's library predates <expected>).
// Header-only; link with libhyle_hip.so and the HIP runtime (amdhip64).  noexcept throughout:
// errors travel as Status, never as exceptions.
#pragma once

#include <hip/hip_runtime_api.h>

#include <array>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <initializer_list>
#include <optional>
#include <span>
#include <string>
#include <utility>
#include <variant>
#include <vector>

#include "hyle_hip.h"

namespace hyle {

// include/hyle/error/status.h:18-44
enum class StatusCode : std::uint16_t {
  Ok = 0, InvalidArgument = 3, ResourceExhausted = 8, FailedPrecondition = 9, OutOfRange = 11,
  Unimplemented = 12, Internal = 13, Unavailable = 14,
};

class Status final {
public:
  Status() noexcept = default;
  Status(StatusCode code, std::string message) noexcept : code_(code), message_(std::move(message)) {}
  static Status Ok() noexcept { return {}; }
  static Status InvalidArgument(std::string m) noexcept { return {StatusCode::InvalidArgument, std::move(m)}; }
  static Status FailedPrecondition(std::string m) noexcept { return {StatusCode::FailedPrecondition, std::move(m)}; }
  static Status OutOfRange(std::string m) noexcept { return {StatusCode::OutOfRange, std::move(m)}; }
  static Status Unimplemented(std::string m) noexcept { return {StatusCode::Unimplemented, std::move(m)}; }
  static Status Internal(std::string m) noexcept { return {StatusCode::Internal, std::move(m)}; }
  static Status Unavailable(std::string m) noexcept { return {StatusCode::Unavailable, std::move(m)}; }
  bool ok() const noexcept { return code_ == StatusCode::Ok; }
  StatusCode code() const noexcept { return code_; }
  const std::string &message() const noexcept { return message_; }
  bool IsInvalidArgument() const noexcept { return code_ == StatusCode::InvalidArgument; }
  bool IsFailedPrecondition() const noexcept { return code_ == StatusCode::FailedPrecondition; }
  bool IsOutOfRange() const noexcept { return code_ == StatusCode::OutOfRange; }
  bool IsUnimplemented() const noexcept { return code_ == StatusCode::Unimplemented; }
  bool IsUnavailable() const noexcept { return code_ == StatusCode::Unavailable; }
  void IgnoreError() const noexcept {}

private:
  StatusCode code_ = StatusCode::Ok;
  std::string message_;
};

// The part of std::expected<T, Status> the reference's call sites use.
template <class T> class Result final {
public:
  Result(T value) noexcept : state_(std::move(value)) {}
  Result(Status error) noexcept : state_(std::move(error)) {}
  bool has_value() const noexcept { return state_.index() == 0; }
  explicit operator bool() const noexcept { return has_value(); }
  T &value() & noexcept { return std::get<0>(state_); }
  const T &value() const & noexcept { return std::get<0>(state_); }
  T &&value() && noexcept { return std::get<0>(std::move(state_)); }
  T &operator*() & noexcept { return std::get<0>(state_); }
  const T &operator*() const & noexcept { return std::get<0>(state_); }
  T &&operator*() && noexcept { return std::get<0>(std::move(state_)); }
  T *operator->() noexcept { return &value(); }
  const T *operator->() const noexcept { return &value(); }
  const Status &error() const noexcept { return std::get<1>(state_); }

private:
  std::variant<T, Status> state_;
};

namespace compute {

namespace detail {
inline Status from_c(hyle_hip_status s) noexcept {
  return s == HYLE_HIP_OK ? Status::Ok() : Status(static_cast<StatusCode>(s), hyle_hip_last_error());
}
inline Status from_hip(hipError_t e, const char *what) noexcept {
  return e == hipSuccess ? Status::Ok() : Status::Internal(std::string(what) + ": " + hipGetErrorString(e));
}
}  // namespace detail

inline constexpr std::size_t kMaxTensorRank = HYLE_HIP_MAX_RANK;

// include/hyle/compute/tensor_desc.h:17-34
enum class DataType : std::uint8_t {
  kUnknown = 0, kBool = 1, kFloat8E4M3FN = 2, kFloat8E5M2 = 3, kFloat16 = 4, kBFloat16 = 5, kFloat32 = 6, kFloat64 = 7,
  kInt8 = 8, kUInt8 = 9, kInt16 = 10, kUInt16 = 11, kInt32 = 12, kUInt32 = 13, kInt64 = 14, kUInt64 = 15,
};
inline std::size_t data_type_size(DataType type) noexcept {
  switch (type) {
    case DataType::kBool: case DataType::kFloat8E4M3FN: case DataType::kFloat8E5M2: case DataType::kInt8:
    case DataType::kUInt8: return 1;
    case DataType::kFloat16: case DataType::kBFloat16: case DataType::kInt16: case DataType::kUInt16: return 2;
    case DataType::kFloat32: case DataType::kInt32: case DataType::kUInt32: return 4;
    case DataType::kFloat64: case DataType::kInt64: case DataType::kUInt64: return 8;
    default: return 0;
  }
}

// include/hyle/compute/tensor_desc.h:141-225
class TensorDesc final {
public:
  TensorDesc() noexcept = default;
  static Result<TensorDesc> dense(DataType type, std::initializer_list<std::int64_t> dims) noexcept {
    return dense(type, dims.begin(), dims.size());
  }
  static Result<TensorDesc> dense(DataType type, const std::int64_t *dims, std::size_t rank) noexcept {
    if (rank > kMaxTensorRank) return Status::InvalidArgument("tensor shape rank exceeds kMaxTensorRank");
    if (data_type_size(type) == 0) return Status::InvalidArgument("tensor data type is invalid");
    TensorDesc d;
    d.c_.dtype = static_cast<std::uint8_t>(type);
    d.c_.rank = static_cast<std::uint8_t>(rank);
    d.c_.elements_per_block = 1;
    bool zero = false;
    for (std::size_t i = 0; i < rank; ++i) {
      if (dims[i] < 0) return Status::InvalidArgument("tensor shape dimension is negative");
      d.c_.dims[i] = dims[i];
      zero = zero || dims[i] == 0;
    }
    if (!zero) {  // a zero extent leaves every stride zero (src/compute_ops/tensor_desc.cc:219-222)
      std::int64_t stride = static_cast<std::int64_t>(data_type_size(type));
      for (std::size_t i = rank; i-- > 0;) {
        d.c_.byte_strides[i] = stride;
        stride *= dims[i];
      }
    }
    return d;
  }
  static Result<TensorDesc> strided_bytes(DataType type, std::initializer_list<std::int64_t> dims,
                                          std::initializer_list<std::int64_t> strides) noexcept {
    if (dims.size() != strides.size()) return Status::InvalidArgument("stride count differs from rank");
    auto d = dense(type, dims);
    if (!d) return d;
    std::size_t i = 0;
    for (std::int64_t s : strides) {
      if (s < 0) return Status::InvalidArgument("negative byte stride");
      d->c_.byte_strides[i++] = s;
    }
    return d;
  }
  // gguf_weight_description(type, logical_type, k, n) (include/hyle/compute/low_precision.h:181-186;
  // block geometry src/compute_ops/low_precision.cc:22-29) for the formats this provider decodes.
  enum class GgufQuantizedType : std::uint8_t { kQ4K = 1, kQ6K = 3, kQ8_0 = 4 };
  static Result<TensorDesc> gguf_weight(GgufQuantizedType type, DataType logical, std::int64_t k,
                                        std::int64_t n) noexcept {
    const std::int64_t per_block = type == GgufQuantizedType::kQ8_0 ? 32 : 256;
    const std::int64_t block_bytes = type == GgufQuantizedType::kQ8_0 ? 34 : (type == GgufQuantizedType::kQ4K ? 144 : 210);
    if (k <= 0 || n <= 0 || k % per_block != 0)
      return Status::InvalidArgument("GGUF weight dimensions do not contain complete K blocks");
    TensorDesc d;
    d.c_.dtype = static_cast<std::uint8_t>(logical);
    d.c_.rank = 2;
    d.c_.storage = HYLE_HIP_STORAGE_BLOCKED;
    d.c_.block_axis = 0;
    d.c_.elements_per_block = static_cast<std::uint32_t>(per_block);
    d.c_.bytes_per_block = static_cast<std::uint32_t>(block_bytes);
    d.c_.dims[0] = k; d.c_.dims[1] = n;
    d.c_.byte_strides[0] = block_bytes; d.c_.byte_strides[1] = k / per_block * block_bytes;
    return d;
  }
  static Result<TensorDesc> gguf_q8_0_weight(DataType logical, std::int64_t k, std::int64_t n) noexcept {
    return gguf_weight(GgufQuantizedType::kQ8_0, logical, k, n);
  }
  bool valid() const noexcept { return c_.dtype != 0; }
  DataType data_type() const noexcept { return static_cast<DataType>(c_.dtype); }
  std::size_t rank() const noexcept { return c_.rank; }
  const std::int64_t *dimensions() const noexcept { return c_.dims; }
  const std::int64_t *byte_strides() const noexcept { return c_.byte_strides; }
  bool is_plain() const noexcept { return c_.storage == HYLE_HIP_STORAGE_PLAIN; }
  bool is_dense() const noexcept {
    if (!is_plain()) return false;
    auto canonical = dense(data_type(), c_.dims, c_.rank);
    return canonical && *canonical == *this;
  }
  std::size_t element_count() const noexcept {
    std::size_t n = 1;
    for (std::size_t i = 0; i < c_.rank; ++i) n *= static_cast<std::size_t>(c_.dims[i]);
    return n;
  }
  std::size_t required_bytes() const noexcept {  // src/compute_ops/tensor_desc.cc:494-540
    if (element_count() == 0) return 0;
    std::size_t last = 0;
    for (std::size_t i = 0; i < c_.rank; ++i) {
      std::size_t units = static_cast<std::size_t>(c_.dims[i]);
      if (!is_plain() && i == c_.block_axis) units /= c_.elements_per_block;
      last += (units - 1) * static_cast<std::size_t>(c_.byte_strides[i]);
    }
    return last + (is_plain() ? data_type_size(data_type()) : c_.bytes_per_block);
  }
  friend bool operator==(const TensorDesc &a, const TensorDesc &b) noexcept {
    if (a.c_.dtype != b.c_.dtype || a.c_.rank != b.c_.rank || a.c_.storage != b.c_.storage) return false;
    for (std::size_t i = 0; i < a.c_.rank; ++i)
      if (a.c_.dims[i] != b.c_.dims[i] || a.c_.byte_strides[i] != b.c_.byte_strides[i]) return false;
    return true;
  }
  friend bool operator!=(const TensorDesc &a, const TensorDesc &b) noexcept { return !(a == b); }
  const hyle_hip_tensor_desc &c_desc() const noexcept { return c_; }
  static TensorDesc from_c(const hyle_hip_tensor_desc &c) noexcept {
    TensorDesc d;
    d.c_ = c;
    return d;
  }

private:
  hyle_hip_tensor_desc c_{};
};

// ---- operations: include/hyle/compute/operation.h:57-126,296-417 ------------------------------
enum class UnaryKind : std::uint8_t { kAbs = 0, kNeg, kExp, kLog, kSqrt, kRsqrt, kTanh, kSigmoid, kRelu, kGelu, kGeluTanh, kSilu, kSoftplus };
enum class BinaryKind : std::uint8_t { kAdd = 0, kSubtract, kMultiply, kDivide, kMinimum, kMaximum };
enum class ReductionKind : std::uint8_t { kSum = 0, kMean, kMinimum, kMaximum };
enum class GatedActivationKind : std::uint8_t { kSilu = 0, kGelu, kGeluTanh };
enum class GatedInputKind : std::uint8_t { kPackedHalves = 0, kSeparate };
enum class SoftmaxKind : std::uint8_t { kSoftmax = 0, kLogSoftmax };
enum class MaskKind : std::uint8_t { kNone = 0, kAdditive, kBoolean };

struct Copy final {};
// Exact scalar payload of Fill (include/hyle/compute/operation.h:187-230): a type and the
// element's bit pattern; low-precision floats come in through from_bits.
class ScalarValue final {
public:
  constexpr ScalarValue() noexcept = default;
  constexpr explicit ScalarValue(bool value) noexcept : type_(DataType::kBool), bits_(value ? 1u : 0u) {}
  constexpr explicit ScalarValue(std::int8_t value) noexcept : type_(DataType::kInt8), bits_(static_cast<std::uint8_t>(value)) {}
  constexpr explicit ScalarValue(std::uint8_t value) noexcept : type_(DataType::kUInt8), bits_(value) {}
  constexpr explicit ScalarValue(std::int32_t value) noexcept : type_(DataType::kInt32), bits_(static_cast<std::uint32_t>(value)) {}
  explicit ScalarValue(float value) noexcept : type_(DataType::kFloat32) {
    std::uint32_t word;
    std::memcpy(&word, &value, sizeof word);
    bits_ = word;
  }
  static constexpr ScalarValue from_bits(DataType type, std::uint64_t bits) noexcept {
    ScalarValue result;
    result.type_ = type;
    result.bits_ = bits;
    return result;
  }
  constexpr bool valid() const noexcept { return type_ != DataType::kUnknown; }
  constexpr DataType data_type() const noexcept { return type_; }
  constexpr std::uint64_t bits() const noexcept { return bits_; }
private:
  DataType type_ = DataType::kUnknown;
  std::uint64_t bits_ = 0;
};
// No inputs: a dense tensor of output_shape whose every element is `value`.
struct Fill final {
  std::vector<std::int64_t> output_shape;
  DataType output_type = DataType::kUnknown;
  ScalarValue value;
};
// Inputs (condition Bool, first, second), broadcast together: first where the condition holds.
struct Select final {};
// Up to four inputs joined along `axis` (include/hyle/compute/operation.h:384-386).  A wider Concat is
// prepared as groups of consecutive inputs: `total` is then the output's whole extent along the axis
// and `start` the extent that precedes the group; both stay 0 when one group is the whole Concat.
struct Concat final {
  std::int32_t axis = 0;
  std::uint64_t total = 0;
  std::uint64_t start = 0;
};
// include/hyle/compute/operation.h:102-105,367-370.  Inputs (source, Int32 / Int64 indices): the
// source with `axis` replaced by the shape of the indices.  With checked bounds an index outside
// the axis leaves the output untouched and fails the Completion with OutOfRange.
enum class IndexBoundsPolicy : std::uint8_t { kChecked = 0, kUnchecked = 1 };
struct Gather final {
  std::int32_t axis = 0;
  IndexBoundsPolicy bounds = IndexBoundsPolicy::kChecked;
};
struct Cast final { DataType output_type = DataType::kUnknown; };
struct Unary final { UnaryKind kind = UnaryKind::kAbs; };
struct Binary final { BinaryKind kind = BinaryKind::kAdd; };
// include/hyle/compute/operation.h:232-247: every axis by default, or an explicit list
// (entries may count from the end; duplicates are refused when the output is inferred).
class Axes final {
public:
  constexpr Axes() noexcept = default;
  static Axes all() noexcept { return {}; }
  static Result<Axes> from(std::span<const std::int32_t> axes) noexcept {
    if (axes.empty()) return Status::InvalidArgument("explicit axis list cannot be empty");
    if (axes.size() > HYLE_HIP_MAX_RANK) return Status::InvalidArgument("axis list exceeds kMaxTensorRank");
    Axes result;
    result.all_ = false;
    result.count_ = static_cast<std::uint8_t>(axes.size());
    for (std::size_t i = 0; i < axes.size(); ++i) {
      if (axes[i] < -HYLE_HIP_MAX_RANK || axes[i] >= HYLE_HIP_MAX_RANK)
        return Status::OutOfRange("axis cannot address a supported tensor rank");
      result.values_[i] = static_cast<std::int8_t>(axes[i]);
    }
    return result;
  }
  constexpr bool is_all() const noexcept { return all_; }
  constexpr std::span<const std::int8_t> values() const noexcept { return {values_.data(), count_}; }

private:
  std::array<std::int8_t, HYLE_HIP_MAX_RANK> values_{};
  std::uint8_t count_ = 0;
  bool all_ = true;
};
struct Reduce final {
  ReductionKind kind = ReductionKind::kSum;
  Axes axes = Axes::all();
  bool keep_dimensions = false;
  DataType accumulation_type = DataType::kUnknown;
};
struct RmsNorm final { float epsilon = 1.0e-5F; DataType accumulation_type = DataType::kFloat32; };
struct LayerNorm final { float epsilon = 1.0e-5F; DataType accumulation_type = DataType::kFloat32; };
struct GatedActivation final {
  GatedActivationKind activation = GatedActivationKind::kSilu;
  GatedInputKind inputs = GatedInputKind::kPackedHalves;
};
struct Softmax final {
  std::int32_t axis = -1;
  float scale = 1.0F;
  SoftmaxKind kind = SoftmaxKind::kSoftmax;
  MaskKind mask = MaskKind::kNone;
  DataType accumulation_type = DataType::kFloat32;
};
struct TopK final { std::size_t count = 1; std::int32_t axis = -1; bool largest = true; bool sorted = true; bool stable = true; };
// Fused forms of this provider (custom operations on the reference side).
struct BinaryChain final { BinaryKind first = BinaryKind::kAdd; BinaryKind second = BinaryKind::kMultiply; };
struct Q8_0DequantSumSquares final {};
// The same operation under its general name (Q8_0, Q4_K or Q6_K weights, told apart by the block
// geometry of the descriptor), and MatMul(x, W) over such a weight for up to 8 activation rows
// (inputs: weight, activations).
using GgufDequantSumSquares = Q8_0DequantSumSquares;
// kGgmlQ8: the activations are first quantised to ggml's 8-bit blocks and the block dots are
// integers, as the reference's ggml route computes the product; kExact: exact weights times f32.
enum class ActivationArithmetic : std::uint8_t { kExact = 0, kGgmlQ8 = 1 };
struct GgufMatVec final { ActivationArithmetic activations = ActivationArithmetic::kExact; };

// include/hyle/compute/operation.h:112-115,388-392.  Inputs (data, Int32 / Int64 positions, F32 frequencies).
enum class RopeLayout : std::uint8_t { kInterleaved = 0, kHalfSplit = 1 };
struct RoPE final {
  std::size_t rotary_dimensions = 0;
  std::int32_t sequence_axis = -2;
  RopeLayout layout = RopeLayout::kInterleaved;
};
// sampling_ops::RandomBits / Categorical (include/hyle/compute/sampling_ops.h:12-75)
struct RandomBits final { std::uint32_t word_count = 4; };
struct Categorical final { bool return_log_probability = false; };

using Operation = std::variant<Copy, Fill, Select, Concat, Gather, Cast, Unary, Binary, Reduce, RmsNorm, LayerNorm, GatedActivation, Softmax, TopK, BinaryChain,
                               Q8_0DequantSumSquares, GgufMatVec, RandomBits, Categorical, RoPE>;

namespace detail {
inline hyle_hip_op_desc to_c(const Operation &operation, const TensorDesc *inputs, std::size_t count) noexcept {
  hyle_hip_op_desc r{};
  r.abi_version = HYLE_HIP_ABI_VERSION;
  r.scale = 1.0F;
  r.largest = 1;
  struct Fill {
    hyle_hip_op_desc &r;
    void operator()(const Copy &) const { r.op = HYLE_HIP_OP_COPY; }
    void operator()(const compute::Fill &o) const {
      // the scalar's type travels as the output type; a scalar of another type is made invalid here
      // so that the schema refuses it (src/compute_ops/operation.cc:1263-1275)
      r.op = HYLE_HIP_OP_FILL;
      r.kind = o.value.data_type() == o.output_type ? static_cast<std::uint32_t>(o.output_type) : 0u;
      r.count = o.value.bits();
      r.inputs[0].rank = static_cast<std::uint8_t>(o.output_shape.size() <= kMaxTensorRank ? o.output_shape.size() : 255);
      for (std::size_t i = 0; i < o.output_shape.size() && i < kMaxTensorRank; ++i) r.inputs[0].dims[i] = o.output_shape[i];
    }
    void operator()(const Select &) const { r.op = HYLE_HIP_OP_SELECT; }
    void operator()(const Concat &o) const {
      r.op = HYLE_HIP_OP_CONCAT; r.axis = o.axis; r.kind = static_cast<std::uint32_t>(o.total); r.count = o.start;
    }
    void operator()(const Gather &o) const {
      r.op = HYLE_HIP_OP_GATHER; r.axis = o.axis; r.kind2 = static_cast<std::uint32_t>(o.bounds);
    }
    void operator()(const Cast &o) const { r.op = HYLE_HIP_OP_CAST; r.kind = static_cast<std::uint32_t>(o.output_type); }
    void operator()(const Unary &o) const { r.op = HYLE_HIP_OP_UNARY; r.kind = static_cast<std::uint32_t>(o.kind); }
    void operator()(const Binary &o) const { r.op = HYLE_HIP_OP_BINARY; r.kind = static_cast<std::uint32_t>(o.kind); }
    void operator()(const Reduce &o) const {
      r.op = HYLE_HIP_OP_REDUCE; r.kind = static_cast<std::uint32_t>(o.kind);
      r.axes_count = o.axes.is_all() ? 0u : static_cast<std::uint32_t>(o.axes.values().size());
      for (std::uint32_t i = 0; i < r.axes_count; ++i) r.axes[i] = o.axes.values()[i];
      r.keep_dimensions = o.keep_dimensions; r.accumulation = static_cast<std::uint32_t>(o.accumulation_type);
    }
    void operator()(const RmsNorm &o) const {
      r.op = HYLE_HIP_OP_RMS_NORM; r.epsilon = o.epsilon; r.accumulation = static_cast<std::uint32_t>(o.accumulation_type);
    }
    void operator()(const LayerNorm &o) const {
      r.op = HYLE_HIP_OP_LAYER_NORM; r.epsilon = o.epsilon; r.accumulation = static_cast<std::uint32_t>(o.accumulation_type);
    }
    void operator()(const GatedActivation &o) const {
      r.op = HYLE_HIP_OP_GATED_ACTIVATION; r.kind = static_cast<std::uint32_t>(o.activation);
      r.kind2 = static_cast<std::uint32_t>(o.inputs);
    }
    void operator()(const Softmax &o) const {
      r.op = HYLE_HIP_OP_SOFTMAX; r.axis = o.axis; r.scale = o.scale; r.kind2 = static_cast<std::uint32_t>(o.kind);
      r.mask = static_cast<std::uint32_t>(o.mask); r.accumulation = static_cast<std::uint32_t>(o.accumulation_type);
    }
    void operator()(const TopK &o) const { r.op = HYLE_HIP_OP_TOP_K; r.count = o.count; r.axis = o.axis; r.largest = o.largest; }
    void operator()(const BinaryChain &o) const {
      r.op = HYLE_HIP_OP_BINARY_CHAIN; r.kind = static_cast<std::uint32_t>(o.first); r.kind2 = static_cast<std::uint32_t>(o.second);
    }
    void operator()(const Q8_0DequantSumSquares &) const { r.op = HYLE_HIP_OP_Q8_0_DEQUANT_SUMSQ; }
    void operator()(const GgufMatVec &o) const { r.op = HYLE_HIP_OP_GGUF_MATVEC; r.kind2 = static_cast<std::uint32_t>(o.activations); }
    void operator()(const RoPE &o) const {
      r.op = HYLE_HIP_OP_ROPE; r.count = o.rotary_dimensions; r.axis = o.sequence_axis; r.kind2 = static_cast<std::uint32_t>(o.layout);
    }
    void operator()(const RandomBits &o) const { r.op = HYLE_HIP_OP_RANDOM_BITS; r.count = o.word_count; }
    void operator()(const Categorical &o) const { r.op = HYLE_HIP_OP_CATEGORICAL; r.kind2 = o.return_log_probability ? 1u : 0u; }
  };
  std::visit(Fill{r}, operation);
  r.input_count = static_cast<std::uint32_t>(count);
  for (std::size_t i = 0; i < count && i < HYLE_HIP_MAX_INPUTS; ++i) r.inputs[i] = inputs[i].c_desc();
  return r;
}
}  // namespace detail

// hyle::compute::infer_output_descriptions (src/compute_ops/operation.cc:1214-1704)
inline Result<std::vector<TensorDesc>> infer_output_descriptions(const Operation &operation,
                                                                 const std::vector<TensorDesc> &inputs) noexcept {
  if (inputs.size() > HYLE_HIP_MAX_INPUTS)
    return Status::InvalidArgument("operation input count does not match its typed contract");
  const hyle_hip_op_desc request = detail::to_c(operation, inputs.data(), inputs.size());
  hyle_hip_tensor_desc outs[HYLE_HIP_MAX_OUTPUTS];
  std::uint32_t count = 0;
  Status status = detail::from_c(hyle_hip_infer_outputs(&request, outs, &count));
  if (!status.ok()) return status;
  std::vector<TensorDesc> result;
  for (std::uint32_t i = 0; i < count; ++i) result.push_back(TensorDesc::from_c(outs[i]));
  return result;
}

// ---- device, memory, queue, completion (a minimal HIP backend) ---------------------------------
namespace hip {
struct Device final { int ordinal = 0; };
inline Device device(int ordinal) noexcept { return Device{ordinal}; }
}  // namespace hip

// Device allocation with host copies: the role mem::Buffer plays in the reference's tests.
class DeviceBuffer final {
public:
  DeviceBuffer() noexcept = default;
  DeviceBuffer(DeviceBuffer &&o) noexcept : data_(o.data_), size_(o.size_) { o.data_ = nullptr; o.size_ = 0; }
  DeviceBuffer &operator=(DeviceBuffer &&o) noexcept {
    if (this != &o) { release(); data_ = o.data_; size_ = o.size_; o.data_ = nullptr; o.size_ = 0; }
    return *this;
  }
  DeviceBuffer(const DeviceBuffer &) = delete;
  DeviceBuffer &operator=(const DeviceBuffer &) = delete;
  ~DeviceBuffer() { release(); }
  static Result<DeviceBuffer> create(std::size_t bytes) noexcept {
    DeviceBuffer b;
    if (bytes != 0) {
      Status s = detail::from_hip(hipMalloc(&b.data_, bytes), "hipMalloc");
      if (!s.ok()) return s;
    }
    b.size_ = bytes;
    return b;
  }
  Status write(const void *host, std::size_t bytes) noexcept {
    if (bytes > size_) return Status::InvalidArgument("write exceeds the buffer");
    return bytes == 0 ? Status::Ok() : detail::from_hip(hipMemcpy(data_, host, bytes, hipMemcpyHostToDevice), "hipMemcpy");
  }
  Status read(void *host, std::size_t bytes) const noexcept {
    if (bytes > size_) return Status::InvalidArgument("read exceeds the buffer");
    return bytes == 0 ? Status::Ok() : detail::from_hip(hipMemcpy(host, data_, bytes, hipMemcpyDeviceToHost), "hipMemcpy");
  }
  void *data() const noexcept { return data_; }
  std::size_t size() const noexcept { return size_; }

private:
  void release() noexcept { if (data_ != nullptr) (void)hipFree(data_); data_ = nullptr; }
  void *data_ = nullptr;
  std::size_t size_ = 0;
};

// include/hyle/compute/tensor.h: a descriptor bound to storage; storage must hold required_bytes().
class ConstTensorView final {
public:
  static Result<ConstTensorView> create(const TensorDesc &desc, const void *data, std::size_t bytes) noexcept {
    if (bytes < desc.required_bytes()) return Status::InvalidArgument("storage is smaller than the tensor needs");
    ConstTensorView v; v.desc_ = desc; v.data_ = data; return v;
  }
  static Result<ConstTensorView> create(const TensorDesc &desc, const DeviceBuffer &buffer) noexcept {
    return create(desc, buffer.data(), buffer.size());
  }
  const TensorDesc &description() const noexcept { return desc_; }
  const void *data() const noexcept { return data_; }
private:
  TensorDesc desc_; const void *data_ = nullptr;
};
class TensorView final {
public:
  static Result<TensorView> create(const TensorDesc &desc, void *data, std::size_t bytes) noexcept {
    if (bytes < desc.required_bytes()) return Status::InvalidArgument("storage is smaller than the tensor needs");
    TensorView v; v.desc_ = desc; v.data_ = data; return v;
  }
  static Result<TensorView> create(const TensorDesc &desc, const DeviceBuffer &buffer) noexcept {
    return create(desc, buffer.data(), buffer.size());
  }
  ConstTensorView as_const() const noexcept { return *ConstTensorView::create(desc_, data_, desc_.required_bytes()); }
  const TensorDesc &description() const noexcept { return desc_; }
  void *data() const noexcept { return data_; }
private:
  TensorDesc desc_; void *data_ = nullptr;
};

// include/hyle/compute/completion.h:40: the event recorded when a sequence finishes.
class Completion final {
public:
  explicit Completion(hipEvent_t event) noexcept : event_(event) {}
  // A launch whose kernels can refuse their input (checked Gather): the plan's status word in
  // `workspace` is read once the event has passed.
  Completion(hipEvent_t event, const hyle_hip_plan *plan, const void *workspace, hipStream_t stream) noexcept
      : event_(event), plan_(plan), workspace_(workspace), stream_(stream) {}
  Completion(Completion &&o) noexcept : event_(o.event_), plan_(o.plan_), workspace_(o.workspace_), stream_(o.stream_) {
    o.event_ = nullptr;
  }
  Completion &operator=(Completion &&o) noexcept {
    std::swap(event_, o.event_); plan_ = o.plan_; workspace_ = o.workspace_; stream_ = o.stream_;
    return *this;
  }
  Completion(const Completion &) = delete;
  ~Completion() { if (event_ != nullptr) (void)hipEventDestroy(event_); }
  Status wait() noexcept {
    if (event_ == nullptr) return Status::Ok();
    Status s = detail::from_hip(hipEventSynchronize(event_), "hipEventSynchronize");
    if (!s.ok() || plan_ == nullptr) return s;
    return detail::from_c(hyle_hip_plan_device_status(plan_, workspace_, stream_));
  }
private:
  hipEvent_t event_ = nullptr;
  const hyle_hip_plan *plan_ = nullptr;
  const void *workspace_ = nullptr;
  hipStream_t stream_ = nullptr;
};

class Queue final {  // one HIP stream (src/compute_backend_cuda: stream-per-Queue)
public:
  explicit Queue(hipStream_t stream) noexcept : stream_(stream) {}
  Queue(Queue &&o) noexcept : stream_(o.stream_) { o.stream_ = nullptr; }
  Queue &operator=(Queue &&o) noexcept { std::swap(stream_, o.stream_); return *this; }
  Queue(const Queue &) = delete;
  ~Queue() { if (stream_ != nullptr) (void)hipStreamDestroy(stream_); }
  hipStream_t stream() const noexcept { return stream_; }
  Status drain() noexcept { return detail::from_hip(hipStreamSynchronize(stream_), "hipStreamSynchronize"); }
private:
  hipStream_t stream_ = nullptr;
};

class Context final {
public:
  Context(Context &&o) noexcept : handle_(o.handle_) { o.handle_ = nullptr; }
  Context &operator=(Context &&o) noexcept { std::swap(handle_, o.handle_); return *this; }
  Context(const Context &) = delete;
  ~Context() { hyle_hip_context_destroy(handle_); }
  static Result<Context> create(hip::Device device) noexcept {
    hyle_hip_context *handle = nullptr;
    Status s = detail::from_c(hyle_hip_context_create(device.ordinal, &handle));
    if (!s.ok()) return s;
    return Context(handle);
  }
  // No device: operations can be prepared and inspected (cold path), never submitted.
  static Context planning_only() noexcept { return Context(nullptr); }
  Result<Queue> create_queue() noexcept {
    if (handle_ == nullptr) return Status::FailedPrecondition("context has no device");
    hipStream_t stream = nullptr;
    Status s = detail::from_hip(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking), "hipStreamCreate");
    if (!s.ok()) return s;
    return Queue(stream);
  }
  hyle_hip_context *handle() const noexcept { return handle_; }
private:
  explicit Context(hyle_hip_context *handle) noexcept : handle_(handle) {}
  hyle_hip_context *handle_ = nullptr;
};

struct WorkspaceRequirement final { std::size_t size = 0; std::size_t alignment = 1; };
struct AliasSupport final { bool supported = false; std::size_t byte_offset = 0; };

class OperationInvocation;

// include/hyle/compute/prepared_operation.h:144-291
class PreparedOperation final {
public:
  PreparedOperation(PreparedOperation &&o) noexcept : plan_(o.plan_) { o.plan_ = nullptr; }
  PreparedOperation &operator=(PreparedOperation &&o) noexcept { std::swap(plan_, o.plan_); return *this; }
  PreparedOperation(const PreparedOperation &) = delete;
  ~PreparedOperation() { hyle_hip_plan_destroy(plan_); }
  Result<TensorDesc> output_description(std::size_t index = 0) const noexcept {
    hyle_hip_tensor_desc outs[HYLE_HIP_MAX_OUTPUTS];
    std::uint32_t count = 0;
    Status s = detail::from_c(hyle_hip_plan_outputs(plan_, outs, &count));
    if (!s.ok()) return s;
    if (index >= count) return Status::InvalidArgument("output index is out of range");
    return TensorDesc::from_c(outs[index]);
  }
  WorkspaceRequirement workspace_requirement() const noexcept {
    WorkspaceRequirement w;
    (void)hyle_hip_plan_workspace(plan_, &w.size, &w.alignment);
    return w;
  }
  Result<AliasSupport> alias_support(std::size_t output, std::size_t input) const noexcept {
    return AliasSupport{hyle_hip_plan_alias_support(plan_, static_cast<std::uint32_t>(output),
                                                    static_cast<std::uint32_t>(input)) != 0, 0};
  }
  std::uint32_t dispatch_count() const noexcept { return hyle_hip_plan_dispatch_count(plan_); }
  const char *route_name() const noexcept { return hyle_hip_plan_route_name(plan_); }
  // The workspace is caller-owned device memory of at least workspace_requirement().size bytes.
  Result<OperationInvocation> create_invocation(void *workspace = nullptr, std::size_t workspace_size = 0) const noexcept;
  const hyle_hip_plan *plan() const noexcept { return plan_; }
  explicit PreparedOperation(hyle_hip_plan *plan) noexcept : plan_(plan) {}
private:
  hyle_hip_plan *plan_ = nullptr;
};

class OperationInvocation final {
public:
  OperationInvocation(const hyle_hip_plan *plan, void *workspace, std::size_t size) noexcept
      : plan_(plan), workspace_(workspace), workspace_size_(size) {}
  // Enqueue on the queue's stream and return a Completion for it; never blocks.  A rejected
  // submission (EnqueueResult::rejected, include/hyle/compute/detail/queue_sequence.h:36-53)
  // leaves the invocation reusable and surfaces as the error Status.
  Result<Completion> submit(Queue &queue, std::initializer_list<ConstTensorView> inputs,
                            std::initializer_list<TensorView> outputs) noexcept {
    const void *in[HYLE_HIP_MAX_INPUTS] = {};
    void *out[HYLE_HIP_MAX_OUTPUTS] = {};
    if (inputs.size() > HYLE_HIP_MAX_INPUTS || outputs.size() > HYLE_HIP_MAX_OUTPUTS)
      return Status::InvalidArgument("too many bindings");
    std::size_t i = 0;
    for (const ConstTensorView &v : inputs) in[i++] = v.data();
    i = 0;
    for (const TensorView &v : outputs) out[i++] = v.data();
    Status s = detail::from_c(hyle_hip_plan_launch(plan_, in, static_cast<std::uint32_t>(inputs.size()), out,
                                                   static_cast<std::uint32_t>(outputs.size()), workspace_,
                                                   workspace_size_, queue.stream()));
    if (!s.ok()) return s;
    hipEvent_t event = nullptr;
    s = detail::from_hip(hipEventCreateWithFlags(&event, hipEventDisableTiming), "hipEventCreate");
    if (!s.ok()) return s;
    s = detail::from_hip(hipEventRecord(event, queue.stream()), "hipEventRecord");
    if (!s.ok()) { (void)hipEventDestroy(event); return s; }
    if (hyle_hip_plan_device_status_offset(plan_, nullptr)) return Completion(event, plan_, workspace_, queue.stream());
    return Completion(event);
  }
  Result<Completion> submit(Queue &queue, const TensorView &out) noexcept {
    return submit(queue, std::initializer_list<ConstTensorView>{}, {out});
  }
  Result<Completion> submit(Queue &queue, const ConstTensorView &a, const TensorView &out) noexcept {
    return submit(queue, {a}, {out});
  }
  Result<Completion> submit(Queue &queue, const ConstTensorView &a, const ConstTensorView &b,
                            const TensorView &out) noexcept {
    return submit(queue, {a, b}, {out});
  }
  Result<Completion> submit(Queue &queue, const ConstTensorView &a, const ConstTensorView &b, const ConstTensorView &c,
                            const TensorView &out) noexcept {
    return submit(queue, {a, b, c}, {out});
  }
private:
  const hyle_hip_plan *plan_;
  void *workspace_;
  std::size_t workspace_size_;
};

inline Result<OperationInvocation> PreparedOperation::create_invocation(void *workspace,
                                                                        std::size_t workspace_size) const noexcept {
  const WorkspaceRequirement need = workspace_requirement();
  if (need.size != 0 && (workspace == nullptr || workspace_size < need.size))
    return Status::InvalidArgument("workspace is smaller than the plan requires");
  return OperationInvocation(plan_, workspace, workspace_size);
}

// hyle::compute::prepare (include/hyle/compute/prepared_operation.h:313-317).  Unimplemented is
// the clean decline a route table moves past (src/compute/operation.cc:1259-1266).
inline Result<PreparedOperation> prepare(const Context &context, const Operation &operation,
                                         std::initializer_list<TensorDesc> inputs) noexcept {
  if (inputs.size() > HYLE_HIP_MAX_INPUTS)
    return Status::InvalidArgument("operation input count does not match its typed contract");
  const hyle_hip_op_desc request = detail::to_c(operation, inputs.begin(), inputs.size());
  hyle_hip_plan *plan = nullptr;
  Status s = detail::from_c(hyle_hip_plan_create(context.handle(), &request, nullptr, 0, &plan));
  if (!s.ok()) return s;
  return PreparedOperation(plan);
}
inline Result<PreparedOperation> prepare(const Context &c, const Operation &op) noexcept {
  return prepare(c, op, std::initializer_list<TensorDesc>{});
}
inline Result<PreparedOperation> prepare(const Context &c, const Operation &op, const TensorDesc &a) noexcept {
  return prepare(c, op, {a});
}
inline Result<PreparedOperation> prepare(const Context &c, const Operation &op, const TensorDesc &a,
                                         const TensorDesc &b) noexcept {
  return prepare(c, op, {a, b});
}
inline Result<PreparedOperation> prepare(const Context &c, const Operation &op, const TensorDesc &a,
                                         const TensorDesc &b, const TensorDesc &d) noexcept {
  return prepare(c, op, {a, b, d});
}

}  // namespace compute
}  // namespace hyle
