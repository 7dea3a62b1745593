// plan.hip -- the C ABI of include/hyle_hip.h: operator schema (output inference),
// admission of a request into a kernel route (the reference's propose + prepare),
// and the allocation-free launch (shared_submit).  Host code only; the kernels
// live in the sibling .hip files behind kernels.h.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <limits>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "../../include/hyle_hip.h"
#include "kernels.h"

using namespace hyle_hip;

// ---------------------------------------------------------------------------------
// errors
// ---------------------------------------------------------------------------------
namespace {

thread_local char g_error[320] = "";

hyle_hip_status fail(hyle_hip_status status, const char *format, ...) {
  va_list args;
  va_start(args, format);
  vsnprintf(g_error, sizeof g_error, format, args);
  va_end(args);
  return status;
}

hyle_hip_status hip_fail(hipError_t error, const char *what) {
  return fail(HYLE_HIP_INTERNAL, "%s: %s", what, hipGetErrorString(error));
}

// ---------------------------------------------------------------------------------
// launch-shape labels (kernels.h)
// ---------------------------------------------------------------------------------
struct VariantList {
  std::mutex mutex;
  std::vector<std::string *> labels;  // never freed: the texts are handed out as C strings
};
VariantList &variant_list() {
  static VariantList *list = new VariantList;  // outlives every static of the library
  return *list;
}
constexpr int kNotedVariants = 4;  // dispatches of one launch
thread_local const char *g_noted[kNotedVariants];
thread_local int g_noted_count = 0;
thread_local char g_noted_text[512];

// ---------------------------------------------------------------------------------
// descriptors
// ---------------------------------------------------------------------------------
typedef hyle_hip_tensor_desc Desc;

size_t dtype_size(uint8_t dtype) {
  switch (dtype) {
    case HYLE_HIP_DTYPE_BOOL:
    case HYLE_HIP_DTYPE_F8_E4M3FN:
    case HYLE_HIP_DTYPE_F8_E5M2:
    case HYLE_HIP_DTYPE_I8:
    case HYLE_HIP_DTYPE_U8: return 1;
    case HYLE_HIP_DTYPE_F16:
    case HYLE_HIP_DTYPE_BF16:
    case HYLE_HIP_DTYPE_I16:
    case HYLE_HIP_DTYPE_U16: return 2;
    case HYLE_HIP_DTYPE_F32:
    case HYLE_HIP_DTYPE_I32:
    case HYLE_HIP_DTYPE_U32: return 4;
    case HYLE_HIP_DTYPE_F64:
    case HYLE_HIP_DTYPE_I64:
    case HYLE_HIP_DTYPE_U64: return 8;
    default: return 0;
  }
}
bool is_index(uint8_t dtype) { return dtype == HYLE_HIP_DTYPE_I32 || dtype == HYLE_HIP_DTYPE_I64; }
// The schema's type classes (src/compute_ops/operation.cc:20-56); what the kernels compute in is
// narrower and decided at admission (to_elem).
bool is_floating(uint8_t dtype) {
  return dtype == HYLE_HIP_DTYPE_F8_E4M3FN || dtype == HYLE_HIP_DTYPE_F8_E5M2 || dtype == HYLE_HIP_DTYPE_F16 ||
         dtype == HYLE_HIP_DTYPE_BF16 || dtype == HYLE_HIP_DTYPE_F32 || dtype == HYLE_HIP_DTYPE_F64;
}
bool is_numeric(uint8_t dtype) {
  return is_floating(dtype) || (dtype >= HYLE_HIP_DTYPE_I8 && dtype <= HYLE_HIP_DTYPE_U64);
}
bool to_elem(uint8_t dtype, Elem *out) {
  switch (dtype) {
    case HYLE_HIP_DTYPE_F32: *out = Elem::kF32; return true;
    case HYLE_HIP_DTYPE_F16: *out = Elem::kF16; return true;
    case HYLE_HIP_DTYPE_BF16: *out = Elem::kBF16; return true;
    default: return false;
  }
}

bool has_zero_extent(const Desc &d) {
  for (int i = 0; i < d.rank; ++i)
    if (d.dims[i] == 0) return true;
  return false;
}

// element count with overflow check; false on overflow
bool element_count(const Desc &d, uint64_t *count) {
  if (has_zero_extent(d)) {
    *count = 0;
    return true;
  }
  uint64_t n = 1;
  for (int i = 0; i < d.rank; ++i) {
    const uint64_t e = (uint64_t)d.dims[i];
    if (e != 0 && n > std::numeric_limits<uint64_t>::max() / e) return false;
    n *= e;
  }
  *count = n;
  return true;
}

// TensorDesc::dense of the reference (src/compute_ops/tensor_desc.cc:211-243): canonical
// row-major byte strides; a shape with a zero extent gets all-zero strides.
hyle_hip_status make_dense(uint8_t dtype, const int64_t *dims, int rank, Desc *out) {
  if (rank < 0 || rank > HYLE_HIP_MAX_RANK)
    return fail(HYLE_HIP_INVALID_ARGUMENT, "tensor shape rank exceeds kMaxTensorRank");
  if (dtype_size(dtype) == 0) return fail(HYLE_HIP_INVALID_ARGUMENT, "tensor data type is invalid");
  std::memset(out, 0, sizeof *out);
  out->dtype = dtype;
  out->rank = (uint8_t)rank;
  out->storage = HYLE_HIP_STORAGE_PLAIN;
  out->elements_per_block = 1;
  bool zero = false;
  for (int i = 0; i < rank; ++i) {
    if (dims[i] < 0) return fail(HYLE_HIP_INVALID_ARGUMENT, "tensor shape dimension is negative");
    out->dims[i] = dims[i];
    zero = zero || dims[i] == 0;
  }
  if (zero) return HYLE_HIP_OK;
  uint64_t stride = dtype_size(dtype);
  for (int i = rank - 1; i >= 0; --i) {
    if (stride > (uint64_t)std::numeric_limits<int64_t>::max())
      return fail(HYLE_HIP_OUT_OF_RANGE, "dense tensor byte stride overflows");
    out->byte_strides[i] = (int64_t)stride;
    const uint64_t e = (uint64_t)dims[i];
    if (e != 0 && stride > std::numeric_limits<uint64_t>::max() / e)
      return fail(HYLE_HIP_OUT_OF_RANGE, "dense tensor byte stride overflows size_t");
    stride *= e;
  }
  return HYLE_HIP_OK;
}

bool same_desc(const Desc &a, const Desc &b) {
  if (a.dtype != b.dtype || a.rank != b.rank || a.storage != b.storage) return false;
  if (a.storage == HYLE_HIP_STORAGE_BLOCKED &&
      (a.block_axis != b.block_axis || a.elements_per_block != b.elements_per_block ||
       a.bytes_per_block != b.bytes_per_block))
    return false;
  for (int i = 0; i < a.rank; ++i)
    if (a.dims[i] != b.dims[i] || a.byte_strides[i] != b.byte_strides[i]) return false;
  return true;
}

bool is_plain(const Desc &d) { return d.storage == HYLE_HIP_STORAGE_PLAIN; }

// TensorDesc::is_dense (src/compute_ops/tensor_desc.cc:542-552): exactly the canonical strides.
bool is_dense(const Desc &d) {
  if (!is_plain(d)) return false;
  Desc canonical;
  if (make_dense(d.dtype, d.dims, d.rank, &canonical) != HYLE_HIP_OK) return false;
  return same_desc(canonical, d);
}

// validate_description of the reference: known type, bounded rank, non-negative extents and
// strides (negative strides are outside the public contract, tensor_desc.h:136-139).
hyle_hip_status validate_desc(const Desc &d, const char *what) {
  if (d.rank > HYLE_HIP_MAX_RANK)
    return fail(HYLE_HIP_INVALID_ARGUMENT, "%s: rank exceeds kMaxTensorRank", what);
  if (dtype_size(d.dtype) == 0)
    return fail(HYLE_HIP_INVALID_ARGUMENT, "%s: data type is invalid", what);
  if (d.storage != HYLE_HIP_STORAGE_PLAIN && d.storage != HYLE_HIP_STORAGE_BLOCKED)
    return fail(HYLE_HIP_INVALID_ARGUMENT, "%s: storage format kind is invalid", what);
  for (int i = 0; i < d.rank; ++i) {
    if (d.dims[i] < 0) return fail(HYLE_HIP_INVALID_ARGUMENT, "%s: dimension is negative", what);
    if (d.byte_strides[i] < 0)
      return fail(HYLE_HIP_INVALID_ARGUMENT, "%s: negative byte stride", what);
  }
  if (d.storage == HYLE_HIP_STORAGE_BLOCKED) {
    if (d.elements_per_block == 0 || d.bytes_per_block == 0)
      return fail(HYLE_HIP_INVALID_ARGUMENT, "%s: blocked storage needs non-zero block geometry",
                  what);
    if (d.block_axis >= d.rank)
      return fail(HYLE_HIP_INVALID_ARGUMENT, "%s: block axis is outside the tensor rank", what);
    if (d.dims[d.block_axis] % d.elements_per_block != 0)
      return fail(HYLE_HIP_INVALID_ARGUMENT, "%s: block axis does not hold whole blocks", what);
  }
  uint64_t count;
  if (!element_count(d, &count))
    return fail(HYLE_HIP_OUT_OF_RANGE, "%s: element count overflows size_t", what);
  return HYLE_HIP_OK;
}

// broadcast_shape (src/compute_ops/operation.cc:249-278)
hyle_hip_status broadcast_shape(const int64_t *l, int lr, const int64_t *r, int rr, int64_t *out,
                                int *out_rank) {
  const int rank = lr > rr ? lr : rr;
  if (rank > HYLE_HIP_MAX_RANK)
    return fail(HYLE_HIP_INVALID_ARGUMENT, "broadcast result rank exceeds limit");
  for (int rev = 0; rev < rank; ++rev) {
    const int64_t a = rev < lr ? l[lr - 1 - rev] : 1;
    const int64_t b = rev < rr ? r[rr - 1 - rev] : 1;
    int64_t e;
    if (a == b) e = a;
    else if (a == 1) e = b;
    else if (b == 1) e = a;
    else return fail(HYLE_HIP_INVALID_ARGUMENT, "tensor dimensions cannot be broadcast");
    out[rank - 1 - rev] = e;
  }
  *out_rank = rank;
  return HYLE_HIP_OK;
}

// normalize_axis (src/compute_ops/operation.cc:228-243)
hyle_hip_status normalize_axis(int32_t axis, int rank, int *out) {
  if (rank == 0) return fail(HYLE_HIP_OUT_OF_RANGE, "operation axis requires rank >= 1");
  const int64_t n = axis < 0 ? (int64_t)rank + axis : (int64_t)axis;
  if (n < 0 || n >= rank) return fail(HYLE_HIP_OUT_OF_RANGE, "operation axis is outside tensor rank");
  *out = (int)n;
  return HYLE_HIP_OK;
}

// Reduce::axes as a bit set (src/compute_ops/operation.cc:1358-1377; Axes::from,
// src/compute_ops/operation.cc:768-789): no entries = every axis, a duplicate is refused.
hyle_hip_status reduce_axes(const hyle_hip_op_desc &r, int rank, uint32_t *mask) {
  *mask = 0;
  if (r.axes_count == 0) {
    *mask = (1u << rank) - 1u;
    return HYLE_HIP_OK;
  }
  if (r.axes_count > HYLE_HIP_MAX_RANK)
    return fail(HYLE_HIP_INVALID_ARGUMENT, "axis list exceeds kMaxTensorRank");
  for (uint32_t i = 0; i < r.axes_count; ++i) {
    if (r.axes[i] < -HYLE_HIP_MAX_RANK || r.axes[i] >= HYLE_HIP_MAX_RANK)
      return fail(HYLE_HIP_OUT_OF_RANGE, "axis cannot address a supported tensor rank");
    int axis;
    hyle_hip_status s = normalize_axis(r.axes[i], rank, &axis);
    if (s != HYLE_HIP_OK) return s;
    if ((*mask >> axis) & 1u)
      return fail(HYLE_HIP_INVALID_ARGUMENT, "Reduce axis list contains a duplicate");
    *mask |= 1u << axis;
  }
  return HYLE_HIP_OK;
}

hyle_hip_status validate_accumulation(uint32_t type) {
  if (type == HYLE_HIP_DTYPE_UNKNOWN) return HYLE_HIP_OK;
  if (type > 255 || !is_numeric((uint8_t)type))
    return fail(HYLE_HIP_INVALID_ARGUMENT, "operation accumulation type must be numeric");
  return HYLE_HIP_OK;
}

// ---------------------------------------------------------------------------------
// schema: output inference (src/compute_ops/operation.cc:1214-1704)
// ---------------------------------------------------------------------------------
hyle_hip_status expect_inputs(const hyle_hip_op_desc &r, uint32_t low, uint32_t high) {
  if (r.input_count < low || r.input_count > high || r.input_count > HYLE_HIP_MAX_INPUTS)
    return fail(HYLE_HIP_INVALID_ARGUMENT, "operation input count does not match its typed contract");
  return HYLE_HIP_OK;
}

// gguf_weight_description(type, ..., k, n): logical [K, N], native blocks along axis 0
// (src/compute_ops/low_precision.cc:269-297), for the block geometries this provider decodes
// (src/compute_ops/low_precision.cc:22-29).
hyle_hip_status expect_gguf_weight(const Desc &w) {
  const bool q8_0 = w.elements_per_block == 32 && w.bytes_per_block == 34;
  const bool q4_k = w.elements_per_block == 256 && w.bytes_per_block == 144;
  const bool q6_k = w.elements_per_block == 256 && w.bytes_per_block == 210;
  if (w.storage != HYLE_HIP_STORAGE_BLOCKED || !(q8_0 || q4_k || q6_k) || w.rank != 2 || w.block_axis != 0)
    return fail(HYLE_HIP_INVALID_ARGUMENT,
                "GGUF weight must be blocked [K, N] storage with Q8_0 (32 / 34), Q4_K (256 / 144) or "
                "Q6_K (256 / 210) blocks on axis 0");
  return HYLE_HIP_OK;
}

hyle_hip_status infer(const hyle_hip_op_desc &r, Desc *outs, uint32_t *out_count) {
  if (r.abi_version != HYLE_HIP_ABI_VERSION)
    return fail(HYLE_HIP_INVALID_ARGUMENT, "hyle_hip_op_desc ABI version %u is not %u", r.abi_version,
                HYLE_HIP_ABI_VERSION);
  if (r.input_count > HYLE_HIP_MAX_INPUTS)
    return fail(HYLE_HIP_INVALID_ARGUMENT, "operation input count does not match its typed contract");
  for (uint32_t i = 0; i < r.input_count; ++i) {
    hyle_hip_status s = validate_desc(r.inputs[i], "input");
    if (s != HYLE_HIP_OK) return s;
  }
  const Desc *in = r.inputs;
  hyle_hip_status s;
  *out_count = 1;
  switch (r.op) {
    case HYLE_HIP_OP_COPY: {  // src/compute_ops/operation.cc:1254-1262
      if ((s = expect_inputs(r, 1, 1)) != HYLE_HIP_OK) return s;
      if (!is_plain(in[0]))
        return fail(HYLE_HIP_UNIMPLEMENTED, "Copy handles plain dense/strided storage");
      return make_dense(in[0].dtype, in[0].dims, in[0].rank, &outs[0]);
    }
    case HYLE_HIP_OP_FILL: {  // src/compute_ops/operation.cc:1263-1275
      // no inputs: inputs[0] carries Fill::output_shape (rank, dims), kind the output type, which
      // is also the scalar's type (the two are one field here, so they cannot differ)
      if ((s = expect_inputs(r, 0, 0)) != HYLE_HIP_OK) return s;
      const Desc &shape = r.inputs[0];
      bool valid = shape.rank <= HYLE_HIP_MAX_RANK && r.kind <= 255 && dtype_size((uint8_t)r.kind) != 0;
      for (int i = 0; valid && i < shape.rank; ++i) valid = shape.dims[i] >= 0;
      if (!valid) return fail(HYLE_HIP_INVALID_ARGUMENT, "Fill requires a valid shape and exactly typed scalar");
      return make_dense((uint8_t)r.kind, shape.dims, shape.rank, &outs[0]);
    }
    case HYLE_HIP_OP_SELECT: {  // src/compute_ops/operation.cc:1309-1330
      if ((s = expect_inputs(r, 3, 3)) != HYLE_HIP_OK) return s;
      if (in[0].dtype != HYLE_HIP_DTYPE_BOOL || in[1].dtype != in[2].dtype)
        return fail(HYLE_HIP_INVALID_ARGUMENT, "Select requires Bool condition and equal branch types");
      int64_t branches[HYLE_HIP_MAX_RANK], dims[HYLE_HIP_MAX_RANK];
      int branch_rank, rank;
      if ((s = broadcast_shape(in[1].dims, in[1].rank, in[2].dims, in[2].rank, branches, &branch_rank)) != HYLE_HIP_OK)
        return s;
      if ((s = broadcast_shape(in[0].dims, in[0].rank, branches, branch_rank, dims, &rank)) != HYLE_HIP_OK) return s;
      return make_dense(in[1].dtype, dims, rank, &outs[0]);
    }
    case HYLE_HIP_OP_CONCAT: {  // src/compute_ops/operation.cc:1516-1564
      if ((s = expect_inputs(r, 1, HYLE_HIP_MAX_INPUTS)) != HYLE_HIP_OK) return s;
      int axis;
      if ((s = normalize_axis(r.axis, in[0].rank, &axis)) != HYLE_HIP_OK) return s;
      int64_t dims[HYLE_HIP_MAX_RANK];
      for (int a = 0; a < in[0].rank; ++a) dims[a] = in[0].dims[a];
      for (uint32_t i = 1; i < r.input_count; ++i) {
        if (in[i].dtype != in[0].dtype || in[i].rank != in[0].rank)
          return fail(HYLE_HIP_INVALID_ARGUMENT, "Concat inputs must have equal data type and rank");
        for (int a = 0; a < in[0].rank; ++a)
          if (a != axis && in[i].dims[a] != dims[a])
            return fail(HYLE_HIP_INVALID_ARGUMENT, "Concat non-axis dimensions must match");
        if (in[i].dims[axis] > std::numeric_limits<int64_t>::max() - dims[axis])
          return fail(HYLE_HIP_OUT_OF_RANGE, "Concat axis dimension overflows int64");
        dims[axis] += in[i].dims[axis];
      }
      if (r.kind != 0) {  // one group of a wider Concat: the output's extent and this group's place in it
        if (r.count > r.kind || (uint64_t)dims[axis] > r.kind - r.count)
          return fail(HYLE_HIP_INVALID_ARGUMENT, "Concat group does not fit the output's extent on the axis");
        dims[axis] = (int64_t)r.kind;
      } else if (r.count != 0) {
        return fail(HYLE_HIP_INVALID_ARGUMENT, "Concat group start needs the output's extent on the axis");
      }
      return make_dense(in[0].dtype, dims, in[0].rank, &outs[0]);
    }
    case HYLE_HIP_OP_CAST: {  // src/compute_ops/operation.cc:1276-1285
      if ((s = expect_inputs(r, 1, 1)) != HYLE_HIP_OK) return s;
      if (r.kind > 255 || dtype_size((uint8_t)r.kind) == 0 || !is_plain(in[0]))
        return fail(HYLE_HIP_INVALID_ARGUMENT, "Cast requires a valid destination type and plain input");
      return make_dense((uint8_t)r.kind, in[0].dims, in[0].rank, &outs[0]);
    }
    case HYLE_HIP_OP_UNARY: {
      if ((s = expect_inputs(r, 1, 1)) != HYLE_HIP_OK) return s;
      if (r.kind > 12) return fail(HYLE_HIP_INVALID_ARGUMENT, "Unary kind is invalid");
      const bool broad = r.kind == 0 /*abs*/ || r.kind == 1 /*neg*/ || r.kind == 8 /*relu*/;
      if ((!broad && !is_floating(in[0].dtype)) || (broad && !is_numeric(in[0].dtype)))
        return fail(HYLE_HIP_INVALID_ARGUMENT, "Unary mode does not support the input data type");
      return make_dense(in[0].dtype, in[0].dims, in[0].rank, &outs[0]);
    }
    case HYLE_HIP_OP_BINARY: {
      if ((s = expect_inputs(r, 2, 2)) != HYLE_HIP_OK) return s;
      if (r.kind > HYLE_HIP_BINARY_MAXIMUM)
        return fail(HYLE_HIP_INVALID_ARGUMENT, "Binary kind is invalid");
      if (in[0].dtype != in[1].dtype)
        return fail(HYLE_HIP_INVALID_ARGUMENT, "binary input data types differ");
      int64_t dims[HYLE_HIP_MAX_RANK];
      int rank;
      if ((s = broadcast_shape(in[0].dims, in[0].rank, in[1].dims, in[1].rank, dims, &rank)) != HYLE_HIP_OK)
        return s;
      return make_dense(in[0].dtype, dims, rank, &outs[0]);
    }
    case HYLE_HIP_OP_BINARY_CHAIN: {
      if ((s = expect_inputs(r, 3, 3)) != HYLE_HIP_OK) return s;
      if (r.kind > HYLE_HIP_BINARY_MAXIMUM || r.kind2 > HYLE_HIP_BINARY_MAXIMUM)
        return fail(HYLE_HIP_INVALID_ARGUMENT, "Binary kind is invalid");
      if (in[0].dtype != in[1].dtype || in[0].dtype != in[2].dtype)
        return fail(HYLE_HIP_INVALID_ARGUMENT, "binary input data types differ");
      int64_t first[HYLE_HIP_MAX_RANK], dims[HYLE_HIP_MAX_RANK];
      int first_rank, rank;
      if ((s = broadcast_shape(in[0].dims, in[0].rank, in[1].dims, in[1].rank, first, &first_rank)) != HYLE_HIP_OK)
        return s;
      if ((s = broadcast_shape(first, first_rank, in[2].dims, in[2].rank, dims, &rank)) != HYLE_HIP_OK)
        return s;
      return make_dense(in[0].dtype, dims, rank, &outs[0]);
    }
    case HYLE_HIP_OP_REDUCE: {
      if ((s = expect_inputs(r, 1, 1)) != HYLE_HIP_OK) return s;
      if (r.kind > HYLE_HIP_REDUCE_MAXIMUM)
        return fail(HYLE_HIP_INVALID_ARGUMENT, "Reduce kind is invalid");
      if (!is_numeric(in[0].dtype))
        return fail(HYLE_HIP_INVALID_ARGUMENT, "Reduce requires a numeric input");
      if ((s = validate_accumulation(r.accumulation)) != HYLE_HIP_OK) return s;
      uint32_t selected;
      if ((s = reduce_axes(r, in[0].rank, &selected)) != HYLE_HIP_OK) return s;
      int64_t dims[HYLE_HIP_MAX_RANK];
      int rank = 0;
      for (int a = 0; a < in[0].rank; ++a) {
        if ((selected >> a) & 1u) {
          if (r.keep_dimensions) dims[rank++] = 1;
        } else {
          dims[rank++] = in[0].dims[a];
        }
      }
      return make_dense(in[0].dtype, dims, rank, &outs[0]);
    }
    case HYLE_HIP_OP_RMS_NORM: {
      if ((s = expect_inputs(r, 1, 2)) != HYLE_HIP_OK) return s;
      if (!std::isfinite(r.epsilon) || r.epsilon < 0.0f)
        return fail(HYLE_HIP_INVALID_ARGUMENT, "RMSNorm epsilon must be finite and non-negative");
      if ((s = validate_accumulation(r.accumulation)) != HYLE_HIP_OK) return s;
      if (!is_floating(in[0].dtype) || in[0].rank == 0)
        return fail(HYLE_HIP_INVALID_ARGUMENT,
                    "normalization requires a floating tensor with rank >= 1");
      if (r.input_count == 2) {
        const bool promoted = in[0].dtype != HYLE_HIP_DTYPE_F32 && in[1].dtype == HYLE_HIP_DTYPE_F32;
        if ((!promoted && in[1].dtype != in[0].dtype) || in[1].rank != 1 ||
            in[1].dims[0] != in[0].dims[in[0].rank - 1])
          return fail(HYLE_HIP_INVALID_ARGUMENT,
                      "normalization scale must match the last input dimension");
      }
      return make_dense(in[0].dtype, in[0].dims, in[0].rank, &outs[0]);
    }
    case HYLE_HIP_OP_LAYER_NORM: {  // src/compute_ops/operation.cc:506-536,1410-1424
      if ((s = expect_inputs(r, 1, 3)) != HYLE_HIP_OK) return s;
      if (!std::isfinite(r.epsilon) || r.epsilon < 0.0f)
        return fail(HYLE_HIP_INVALID_ARGUMENT, "LayerNorm epsilon must be finite and non-negative");
      if ((s = validate_accumulation(r.accumulation)) != HYLE_HIP_OK) return s;
      if (!is_floating(in[0].dtype) || in[0].rank == 0)
        return fail(HYLE_HIP_INVALID_ARGUMENT,
                    "normalization requires a floating tensor with rank >= 1");
      for (uint32_t i = 1; i < r.input_count; ++i) {
        const bool promoted = in[0].dtype != HYLE_HIP_DTYPE_F32 && in[i].dtype == HYLE_HIP_DTYPE_F32;
        if ((!promoted && in[i].dtype != in[0].dtype) || in[i].rank != 1 ||
            in[i].dims[0] != in[0].dims[in[0].rank - 1])
          return fail(HYLE_HIP_INVALID_ARGUMENT,
                      i == 1 ? "normalization scale must match the last input dimension"
                             : "LayerNorm bias must match the last input dimension");
      }
      return make_dense(in[0].dtype, in[0].dims, in[0].rank, &outs[0]);
    }
    case HYLE_HIP_OP_GATED_ACTIVATION: {
      if (r.kind > 2 || r.kind2 > HYLE_HIP_GATED_SEPARATE)
        return fail(HYLE_HIP_INVALID_ARGUMENT, "GatedActivation mode is invalid");
      const bool separate = r.kind2 == HYLE_HIP_GATED_SEPARATE;
      if ((s = expect_inputs(r, separate ? 2 : 1, separate ? 2 : 1)) != HYLE_HIP_OK) return s;
      if (!is_floating(in[0].dtype) || in[0].rank == 0)
        return fail(HYLE_HIP_INVALID_ARGUMENT, "GatedActivation requires floating rank >= 1 inputs");
      if (separate) {
        bool same = in[0].dtype == in[1].dtype && in[0].rank == in[1].rank;
        for (int a = 0; same && a < in[0].rank; ++a) same = in[0].dims[a] == in[1].dims[a];
        if (!same)
          return fail(HYLE_HIP_INVALID_ARGUMENT,
                      "separate gate/value tensors must have equal type and shape");
        return make_dense(in[0].dtype, in[0].dims, in[0].rank, &outs[0]);
      }
      if ((in[0].dims[in[0].rank - 1] & 1) != 0)
        return fail(HYLE_HIP_INVALID_ARGUMENT, "packed gate/value last dimension must be even");
      int64_t dims[HYLE_HIP_MAX_RANK];
      for (int a = 0; a < in[0].rank; ++a) dims[a] = in[0].dims[a];
      dims[in[0].rank - 1] /= 2;
      return make_dense(in[0].dtype, dims, in[0].rank, &outs[0]);
    }
    case HYLE_HIP_OP_SOFTMAX: {
      if (r.kind2 > HYLE_HIP_LOG_SOFTMAX || r.mask > HYLE_HIP_MASK_BOOLEAN)
        return fail(HYLE_HIP_INVALID_ARGUMENT, "Softmax mode is invalid");
      const uint32_t want = r.mask == HYLE_HIP_MASK_NONE ? 1 : 2;
      if ((s = expect_inputs(r, want, want)) != HYLE_HIP_OK) return s;
      if (!is_floating(in[0].dtype) || in[0].rank == 0 || !std::isfinite(r.scale))
        return fail(HYLE_HIP_INVALID_ARGUMENT,
                    "Softmax requires floating rank >= 1 input and finite scale");
      int axis;
      if ((s = normalize_axis(r.axis, in[0].rank, &axis)) != HYLE_HIP_OK) return s;
      if ((s = validate_accumulation(r.accumulation)) != HYLE_HIP_OK) return s;
      if (r.mask != HYLE_HIP_MASK_NONE) {
        if (r.mask == HYLE_HIP_MASK_BOOLEAN && in[1].dtype != HYLE_HIP_DTYPE_BOOL)
          return fail(HYLE_HIP_INVALID_ARGUMENT, "boolean mask requires Bool data type");
        if (r.mask == HYLE_HIP_MASK_ADDITIVE && !is_floating(in[1].dtype))
          return fail(HYLE_HIP_INVALID_ARGUMENT, "additive mask requires a floating data type");
        int64_t dims[HYLE_HIP_MAX_RANK];
        int rank;
        if ((s = broadcast_shape(in[1].dims, in[1].rank, in[0].dims, in[0].rank, dims, &rank)) != HYLE_HIP_OK)
          return s;
        bool same = rank == in[0].rank;
        for (int a = 0; same && a < rank; ++a) same = dims[a] == in[0].dims[a];
        if (!same)
          return fail(HYLE_HIP_INVALID_ARGUMENT,
                      "tensor is not broadcast-compatible with target shape");
      }
      return make_dense(in[0].dtype, in[0].dims, in[0].rank, &outs[0]);
    }
    case HYLE_HIP_OP_GATHER: {  // src/compute_ops/operation.cc:112-118,616-637,1470-1489
      if ((s = expect_inputs(r, 2, 2)) != HYLE_HIP_OK) return s;
      if (r.kind2 > HYLE_HIP_BOUNDS_UNCHECKED)
        return fail(HYLE_HIP_INVALID_ARGUMENT, "Gather bounds policy is invalid");
      if (!is_index(in[1].dtype)) return fail(HYLE_HIP_INVALID_ARGUMENT, "Gather indices must use Int32 or Int64");
      int axis;
      if ((s = normalize_axis(r.axis, in[0].rank, &axis)) != HYLE_HIP_OK) return s;
      if (in[0].rank - 1 + in[1].rank > HYLE_HIP_MAX_RANK)
        return fail(HYLE_HIP_INVALID_ARGUMENT, "Gather output rank exceeds limit");
      int64_t dims[HYLE_HIP_MAX_RANK];
      int rank = 0;
      for (int a = 0; a < axis; ++a) dims[rank++] = in[0].dims[a];
      for (int a = 0; a < in[1].rank; ++a) dims[rank++] = in[1].dims[a];
      for (int a = axis + 1; a < in[0].rank; ++a) dims[rank++] = in[0].dims[a];
      return make_dense(in[0].dtype, dims, rank, &outs[0]);
    }
    case HYLE_HIP_OP_ROPE: {  // src/compute_ops/operation.cc:127-132,639-696,1566-1574
      if ((s = expect_inputs(r, 3, 3)) != HYLE_HIP_OK) return s;
      if (r.kind2 > HYLE_HIP_ROPE_HALF_SPLIT) return fail(HYLE_HIP_INVALID_ARGUMENT, "RoPE layout is invalid");
      const Desc &data = in[0], &positions = in[1], &frequencies = in[2];
      if (!is_floating(data.dtype) || !is_floating(frequencies.dtype) || !is_index(positions.dtype))
        return fail(HYLE_HIP_INVALID_ARGUMENT, "RoPE requires floating data/frequencies and i32/i64 positions");
      if (data.rank < 2 || r.count == 0 || (r.count & 1u) != 0 || r.count > (uint64_t)data.dims[data.rank - 1])
        return fail(HYLE_HIP_INVALID_ARGUMENT, "RoPE rotary dimension must be positive, even and fit the last axis");
      int sequence_axis;
      if ((s = normalize_axis(r.axis, data.rank, &sequence_axis)) != HYLE_HIP_OK) return s;
      if (sequence_axis == data.rank - 1)
        return fail(HYLE_HIP_INVALID_ARGUMENT, "RoPE sequence axis cannot be the rotary depth axis");
      const int64_t extent = data.dims[sequence_axis];
      if (positions.rank == 0 || (positions.rank == 1 && positions.dims[0] != extent))
        return fail(HYLE_HIP_INVALID_ARGUMENT, "RoPE positions must include the complete sequence axis");
      if (positions.rank > 1) {
        if (positions.rank != sequence_axis + 1)
          return fail(HYLE_HIP_INVALID_ARGUMENT, "RoPE batched positions must match the data prefix through sequence");
        for (int a = 0; a < positions.rank; ++a)
          if (positions.dims[a] != data.dims[a])
            return fail(HYLE_HIP_INVALID_ARGUMENT, "RoPE batched position shape does not match data prefix");
      }
      if (frequencies.rank == 0 || frequencies.dims[frequencies.rank - 1] != (int64_t)(r.count / 2))
        return fail(HYLE_HIP_INVALID_ARGUMENT, "RoPE frequency last dimension must equal rotary_dimensions / 2");
      if (frequencies.rank > 2 || (frequencies.rank == 2 && frequencies.dims[0] != extent))
        return fail(HYLE_HIP_INVALID_ARGUMENT, "RoPE frequencies must be [pairs] or [sequence,pairs]");
      return make_dense(data.dtype, data.dims, data.rank, &outs[0]);
    }
    case HYLE_HIP_OP_RANDOM_BITS:
    case HYLE_HIP_OP_CATEGORICAL: {  // src/compute_ops/sampling_ops.cc:8-63
      const bool bits = r.op == HYLE_HIP_OP_RANDOM_BITS;
      if ((s = expect_inputs(r, bits ? 1 : 2, bits ? 1 : 2)) != HYLE_HIP_OK) return s;
      const Desc &counters = in[bits ? 0 : 1];
      if (!is_plain(counters) || !is_dense(counters) || counters.dtype != HYLE_HIP_DTYPE_U32 || counters.rank != 2 ||
          counters.dims[1] != 4)
        return fail(HYLE_HIP_INVALID_ARGUMENT, "sampling counters require dense U32[R,4] key/draw words");
      if (bits) {
        if (r.count > (uint64_t)std::numeric_limits<int32_t>::max())
          return fail(HYLE_HIP_OUT_OF_RANGE, "RandomBits word count exceeds I32");
        const int64_t dims[2] = {counters.dims[0], (int64_t)r.count};
        return make_dense(HYLE_HIP_DTYPE_U32, dims, 2, &outs[0]);
      }
      if (r.kind2 > 1) return fail(HYLE_HIP_INVALID_ARGUMENT, "Categorical input/output arity differs");
      const Desc &logits = in[0];
      if (!is_plain(logits) || !is_dense(logits) || logits.rank != 2 ||
          (logits.dtype != HYLE_HIP_DTYPE_F16 && logits.dtype != HYLE_HIP_DTYPE_BF16 && logits.dtype != HYLE_HIP_DTYPE_F32))
        return fail(HYLE_HIP_INVALID_ARGUMENT, "Categorical requires dense F16/BF16/F32[R,V] log-weights");
      if (logits.dims[0] != counters.dims[0])
        return fail(HYLE_HIP_INVALID_ARGUMENT, "Categorical counter row count differs");
      if (logits.dims[1] == 0) return fail(HYLE_HIP_INVALID_ARGUMENT, "Categorical requires positive vocabulary");
      if (logits.dims[1] > (int64_t)std::numeric_limits<int32_t>::max())
        return fail(HYLE_HIP_OUT_OF_RANGE, "Categorical vocabulary exceeds I32 indices");
      const int64_t dims[1] = {logits.dims[0]};
      if ((s = make_dense(HYLE_HIP_DTYPE_I32, dims, 1, &outs[0])) != HYLE_HIP_OK) return s;
      if (r.kind2 == 1) {
        *out_count = 2;
        return make_dense(HYLE_HIP_DTYPE_F32, dims, 1, &outs[1]);
      }
      return HYLE_HIP_OK;
    }
    case HYLE_HIP_OP_TOP_K: {
      if ((s = expect_inputs(r, 1, 1)) != HYLE_HIP_OK) return s;
      if (!is_numeric(in[0].dtype) || in[0].rank == 0)
        return fail(HYLE_HIP_INVALID_ARGUMENT, "TopK requires numeric rank >= 1 input");
      int axis;
      if ((s = normalize_axis(r.axis, in[0].rank, &axis)) != HYLE_HIP_OK) return s;
      if (in[0].dims[axis] > (int64_t)std::numeric_limits<int32_t>::max())
        return fail(HYLE_HIP_OUT_OF_RANGE,
                    "TopK selected dimension cannot be represented by i32 indices");
      if (r.count > (uint64_t)in[0].dims[axis])
        return fail(HYLE_HIP_OUT_OF_RANGE, "TopK count exceeds selected dimension");
      int64_t dims[HYLE_HIP_MAX_RANK];
      for (int a = 0; a < in[0].rank; ++a) dims[a] = in[0].dims[a];
      dims[axis] = (int64_t)r.count;
      if ((s = make_dense(in[0].dtype, dims, in[0].rank, &outs[0])) != HYLE_HIP_OK) return s;
      *out_count = 2;
      return make_dense(HYLE_HIP_DTYPE_I32, dims, in[0].rank, &outs[1]);
    }
    case HYLE_HIP_OP_Q8_0_DEQUANT_SUMSQ: {
      if ((s = expect_inputs(r, 1, 1)) != HYLE_HIP_OK) return s;
      if ((s = expect_gguf_weight(in[0])) != HYLE_HIP_OK) return s;
      if (!is_floating(in[0].dtype))
        return fail(HYLE_HIP_INVALID_ARGUMENT, "GGUF weight requires a floating logical type");
      const int64_t dims0[2] = {in[0].dims[1], in[0].dims[0]};
      if ((s = make_dense(HYLE_HIP_DTYPE_BF16, dims0, 2, &outs[0])) != HYLE_HIP_OK) return s;
      *out_count = 2;
      return make_dense(HYLE_HIP_DTYPE_F32, &in[0].dims[1], 1, &outs[1]);
    }
    case HYLE_HIP_OP_GGUF_MATVEC: {
      if ((s = expect_inputs(r, 2, 2)) != HYLE_HIP_OK) return s;
      if ((s = expect_gguf_weight(in[0])) != HYLE_HIP_OK) return s;
      if (r.kind2 > HYLE_HIP_ACTIVATIONS_GGML_Q8)
        return fail(HYLE_HIP_INVALID_ARGUMENT, "GGUF matvec activation mode is invalid");
      // MatMul contraction (src/compute_ops/operation.cc, kMatMul): the last axis of the
      // activations meets the first logical axis of the weight
      if (!is_floating(in[1].dtype) || in[1].rank < 1 || in[1].rank > 2 ||
          in[1].dims[in[1].rank - 1] != in[0].dims[0])
        return fail(HYLE_HIP_INVALID_ARGUMENT,
                    "activations must be floating [K] or [M, K] with K the weight's first logical extent");
      int64_t dims[2];
      int rank = 0;
      if (in[1].rank == 2) dims[rank++] = in[1].dims[0];
      dims[rank++] = in[0].dims[1];
      return make_dense(in[1].dtype, dims, rank, &outs[0]);
    }
    default:
      return fail(HYLE_HIP_UNIMPLEMENTED, "operation kind %u is not served by this provider", r.op);
  }
}

// ---------------------------------------------------------------------------------
// plans
// ---------------------------------------------------------------------------------
enum class Route : uint8_t {
  kNoOp = 0,
  kEwFlat,
  kEwGeneral,
  kSwigluPacked,
  kRmsNorm,
  kSoftmax,
  kReduce,
  kArgmax,
  kTopK,
  kQ8Dequant,
  kKQuantDequant,
  kGgufMatVec,
  kCast,
  kFill,
  kSelect,
  kConcat,
  kGather,
  kRandomBits,
  kCategorical,
  kRope,
};

const char *route_name(Route r) {
  switch (r) {
    case Route::kNoOp: return "no-op";
    case Route::kEwFlat: return "elementwise-flat";
    case Route::kEwGeneral: return "elementwise-strided";
    case Route::kSwigluPacked: return "swiglu-packed";
    case Route::kRmsNorm: return "norm-rows";
    case Route::kSoftmax: return "softmax-rows";
    case Route::kReduce: return "reduce";
    case Route::kArgmax: return "argmax-tiles";
    case Route::kTopK: return "topk-sorted-tiles";
    case Route::kQ8Dequant: return "q8_0-dequant-rows";
    case Route::kKQuantDequant: return "k-quant-dequant-rows";
    case Route::kGgufMatVec: return "gguf-matvec-rows";
    case Route::kCast: return "cast-copy";
    case Route::kFill: return "fill-pattern";
    case Route::kSelect: return "select";
    case Route::kConcat: return "concat";
    case Route::kGather: return "gather";
    case Route::kRandomBits: return "philox-words";
    case Route::kCategorical: return "categorical-tiles";
    case Route::kRope: return "rope-rows";
  }
  return "?";
}

constexpr uint64_t kMaxElements = (uint64_t)std::numeric_limits<int32_t>::max();

}  // namespace

struct hyle_hip_context {
  int device = 0;
  int compute_units = 0;
  void *static_scratch = nullptr;  // this device's copy of `scratch` (hyle_hip_plan_launch_static)
};

struct hyle_hip_plan {
  const hyle_hip_context *context = nullptr;
  hyle_hip_op_desc request{};
  Desc outputs[HYLE_HIP_MAX_OUTPUTS]{};
  uint32_t output_count = 0;
  Route route = Route::kNoOp;
  Elem elem = Elem::kF32;
  uint8_t alias_inputs[HYLE_HIP_MAX_OUTPUTS] = {0, 0};  // bit i: output may alias input i
  uint32_t dispatches = 0;
  size_t workspace_size = 0, workspace_alignment = 1;
  size_t input_alignment[HYLE_HIP_MAX_INPUTS] = {1, 1, 1, 1};   // element alignment (required)
  size_t output_alignment[HYLE_HIP_MAX_OUTPUTS] = {1, 1};
  uint64_t input_elements[HYLE_HIP_MAX_INPUTS] = {0, 0, 0, 0};
  uint64_t output_elements[HYLE_HIP_MAX_OUTPUTS] = {0, 0};
  // route parameters
  EwFlat flat;
  EwGeneral general;
  EwPacked packed;
  NormParams norm;
  SoftmaxParams softmax;
  SoftmaxGeneralParams softmax_general;
  bool softmax_rows_ok = false;     // the row kernel applies (dense last-axis layout)
  bool softmax_mask_vector_ok = false;
  ReduceParams reduce;
  ArgmaxParams argmax;
  TopKParams topk;
  Q8Params q8;
  KQuantParams kquant;
  MatVecParams matvec;
  CastParams cast;
  FillParams fill;
  SelectParams select;
  ConcatParams concat;
  GatherParams gather;
  RandomBitsParams random_bits;
  CategoricalParams categorical;
  RopeParams rope;
  // Concat and Gather take no alias and no overlap: bytes each input spans, for the launch's check
  uint64_t concat_input_bytes[HYLE_HIP_MAX_INPUTS] = {0, 0, 0, 0};
  // Cast and Copy take no alias at all (AliasPolicy::kNone, src/compute_ops/operation.cc:935-957):
  // the bytes the input and the output occupy must not overlap.
  uint64_t no_overlap_input_bytes = 0, no_overlap_output_bytes = 0;
};

namespace {

bool dims_equal(const Desc &a, const Desc &b) {
  if (a.rank != b.rank) return false;
  for (int i = 0; i < a.rank; ++i)
    if (a.dims[i] != b.dims[i]) return false;
  return true;
}

// A dense input that is a trailing slice of the output shape (leading axes absent or 1):
// it repeats every `period` elements of the flat output
// (dense_broadcast_suffix, src/compute_provider_native/elementwise.cc:540-571).
bool suffix_period(const Desc &in, const Desc &out, uint64_t out_elements, uint32_t *period) {
  if (!is_dense(in)) return false;
  uint64_t count = 1;
  bool leading = false;  // once an axis is broadcast, every axis left of it must be too
  for (int rev = 0; rev < out.rank; ++rev) {
    const int64_t oe = out.dims[out.rank - 1 - rev];
    const int64_t ie = rev < in.rank ? in.dims[in.rank - 1 - rev] : 1;
    if (!leading && ie == oe) {
      count *= (uint64_t)ie;
      continue;
    }
    if (ie != 1) return false;
    leading = true;
  }
  if (count == out_elements) *period = 0;
  else *period = (uint32_t)count;
  return true;
}

hyle_hip_status admit_elementwise(hyle_hip_plan *p, EwOp op, int inputs) {
  const hyle_hip_op_desc &r = p->request;
  const Desc &out = p->outputs[0];
  if (!to_elem(out.dtype, &p->elem))
    return fail(HYLE_HIP_UNIMPLEMENTED, "elementwise arithmetic requires plain float32/float16/bfloat16");
  for (int i = 0; i < inputs; ++i)
    if (!is_plain(r.inputs[i]) || r.inputs[i].dtype != out.dtype)
      return fail(HYLE_HIP_UNIMPLEMENTED, "elementwise arithmetic requires plain float32/float16/bfloat16");
  const uint64_t n = p->output_elements[0];
  if (n > kMaxElements)
    return fail(HYLE_HIP_UNIMPLEMENTED, "elementwise output exceeds INT32_MAX elements");
  if (n == 0) {
    p->route = Route::kNoOp;
    return HYLE_HIP_OK;
  }
  // alias only when an input descriptor equals the output descriptor
  // (src/compute_provider_native/elementwise.cc:645-655; gated routes take no alias)
  if (op != EwOp::kSwiglu && op != EwOp::kGated)
    for (int i = 0; i < inputs; ++i)
      if (same_desc(r.inputs[i], out)) p->alias_inputs[0] |= (uint8_t)(1u << i);

  uint32_t period[3] = {0, 0, 0};
  bool flat = true;
  for (int i = 0; i < inputs && flat; ++i) flat = suffix_period(r.inputs[i], out, n, &period[i]);
  p->dispatches = 1;
  if (flat) {
    p->route = Route::kEwFlat;
    p->flat.elements = n;
    p->flat.op = op;
    p->flat.kind0 = (uint8_t)r.kind;
    p->flat.kind1 = (uint8_t)r.kind2;
    p->flat.inputs = (uint8_t)inputs;
    for (int i = 0; i < 3; ++i) p->flat.period[i] = period[i];
    return HYLE_HIP_OK;
  }
  p->route = Route::kEwGeneral;
  EwGeneral &g = p->general;
  g.elements = n;
  g.rank = out.rank;
  g.op = op;
  g.kind0 = (uint8_t)r.kind;
  g.kind1 = (uint8_t)r.kind2;
  g.inputs = (uint8_t)inputs;
  for (int a = 0; a < out.rank; ++a) g.dims[a] = (uint32_t)out.dims[a];
  for (int i = 0; i < inputs; ++i) {
    const Desc &in = r.inputs[i];
    for (int rev = 0; rev < out.rank; ++rev) {
      const int oa = out.rank - 1 - rev;
      int64_t stride = 0;
      if (rev < in.rank) {
        const int ia = in.rank - 1 - rev;
        // logical_broadcast_byte_offset: an input axis of extent 1 contributes nothing
        if (in.dims[ia] != 1) stride = in.byte_strides[ia];
      }
      g.strides[i][oa] = stride;
    }
  }
  return HYLE_HIP_OK;
}

hyle_hip_status require_f32_accumulation(const hyle_hip_plan *p, uint8_t input_dtype, const char *op) {
  const uint32_t acc = p->request.accumulation;
  if (acc == HYLE_HIP_DTYPE_F32) return HYLE_HIP_OK;
  if (acc == HYLE_HIP_DTYPE_UNKNOWN && input_dtype == HYLE_HIP_DTYPE_F32) return HYLE_HIP_OK;
  return fail(HYLE_HIP_UNIMPLEMENTED, "%s supports float32 accumulation (explicit for half inputs)", op);
}

// Physical layout of a GGUF weight the kernels walk: the blocks of a row one after another, rows
// at least a row of blocks apart, at most INT32_MAX values.
hyle_hip_status admit_gguf_rows(const Desc &w) {
  const int64_t k = w.dims[0], n = w.dims[1];
  const int64_t per_block = w.elements_per_block, block_bytes = w.bytes_per_block;
  if (w.byte_strides[0] != block_bytes)
    return fail(HYLE_HIP_UNIMPLEMENTED, "GGUF blocks of a row must be contiguous (block stride = block bytes)");
  if (k > 0 && n > 1 && w.byte_strides[1] < (k / per_block) * block_bytes)
    return fail(HYLE_HIP_INVALID_ARGUMENT, "GGUF row stride is shorter than a row of blocks");
  if ((uint64_t)k * (uint64_t)n > kMaxElements)
    return fail(HYLE_HIP_UNIMPLEMENTED, "GGUF weights of at most INT32_MAX values are served");
  return HYLE_HIP_OK;
}

hyle_hip_status admit(hyle_hip_plan *p) {
  const hyle_hip_op_desc &r = p->request;
  const Desc *in = r.inputs;
  const Desc &out = p->outputs[0];
  // a plan made without a device is sized for the 256 units of an MI355X
  const uint32_t units = p->context != nullptr && p->context->compute_units > 0 ? (uint32_t)p->context->compute_units : 256u;
  hyle_hip_status s;
  switch (r.op) {
    case HYLE_HIP_OP_UNARY:
      // integer abs / neg / relu pass the schema but are not served (FP32/FP16/BF16 only,
      // include/hyle/compute/providers/cuda.h:20-23)
      return admit_elementwise(p, r.kind == HYLE_HIP_UNARY_SILU ? EwOp::kSilu : EwOp::kUnary, 1);
    case HYLE_HIP_OP_BINARY:
      return admit_elementwise(p, EwOp::kBinary, 2);
    case HYLE_HIP_OP_BINARY_CHAIN:
      return admit_elementwise(p, EwOp::kChain, 3);
    case HYLE_HIP_OP_GATED_ACTIVATION: {
      // SiLU, GELU and GELU-tanh (include/hyle/compute/providers/cuda.h:52-54); dense inputs and output (src/compute_provider_cuda/cuda_provider.cc:86-139)
      for (uint32_t i = 0; i < r.input_count; ++i)
        if (!is_dense(in[i]))
          return fail(HYLE_HIP_UNIMPLEMENTED, "gated activation requires dense plain input");
      if (r.kind2 == HYLE_HIP_GATED_SEPARATE)
        return admit_elementwise(p, r.kind == HYLE_HIP_GATED_SILU ? EwOp::kSwiglu : EwOp::kGated, 2);
      if (!to_elem(out.dtype, &p->elem))
        return fail(HYLE_HIP_UNIMPLEMENTED, "gated activation requires dense FP16/BF16/FP32");
      if (p->output_elements[0] > kMaxElements)
        return fail(HYLE_HIP_UNIMPLEMENTED, "gated activation requires at most INT32_MAX elements");
      if (p->output_elements[0] == 0) return HYLE_HIP_OK;
      p->route = Route::kSwigluPacked;
      p->packed.hidden = (uint32_t)out.dims[out.rank - 1];
      p->packed.rows = p->output_elements[0] / p->packed.hidden;
      p->packed.activation = (uint8_t)r.kind;
      p->dispatches = 1;
      return HYLE_HIP_OK;
    }
    case HYLE_HIP_OP_LAYER_NORM:
    case HYLE_HIP_OP_RMS_NORM: {
      if (r.accumulation != HYLE_HIP_DTYPE_F32)
        return fail(HYLE_HIP_UNIMPLEMENTED, "normalization supports float32 accumulation");
      if (!to_elem(in[0].dtype, &p->elem) || !is_dense(in[0]))
        return fail(HYLE_HIP_UNIMPLEMENTED,
                    "normalization requires dense plain float32/float16/bfloat16");
      for (uint32_t i = 1; i < r.input_count; ++i)
        if (!is_dense(in[i]) || in[i].dtype != in[1].dtype)
          return fail(HYLE_HIP_UNIMPLEMENTED,
                      "normalization requires dense plain parameters of one type");
      if (p->output_elements[0] > kMaxElements)
        return fail(HYLE_HIP_UNIMPLEMENTED, "normalization requires at most INT32_MAX elements");
      p->alias_inputs[0] = 1;  // reductions finish before the first write
      if (p->output_elements[0] == 0) return HYLE_HIP_OK;
      p->route = Route::kRmsNorm;
      p->norm.shape.width = (uint32_t)in[0].dims[in[0].rank - 1];
      p->norm.shape.rows = p->output_elements[0] / p->norm.shape.width;
      p->norm.epsilon = r.epsilon;
      p->norm.layer = r.op == HYLE_HIP_OP_LAYER_NORM;
      p->norm.has_weight = r.input_count >= 2;
      p->norm.has_bias = r.input_count == 3;
      p->norm.weight_f32 = r.input_count >= 2 && in[1].dtype == HYLE_HIP_DTYPE_F32 &&
                           in[0].dtype != HYLE_HIP_DTYPE_F32;
      p->dispatches = 1;
      return HYLE_HIP_OK;
    }
    case HYLE_HIP_OP_SOFTMAX: {
      if (!to_elem(in[0].dtype, &p->elem) || !is_plain(in[0]))
        return fail(HYLE_HIP_UNIMPLEMENTED, "Softmax requires plain float32/float16/bfloat16");
      if ((s = require_f32_accumulation(p, in[0].dtype, "Softmax")) != HYLE_HIP_OK) return s;
      if (r.mask != HYLE_HIP_MASK_NONE) {
        if (!is_plain(in[1]) || (r.mask == HYLE_HIP_MASK_ADDITIVE && in[1].dtype != in[0].dtype))
          return fail(HYLE_HIP_UNIMPLEMENTED,
                      "Softmax requires plain Bool or matching floating masks");
      }
      if (p->output_elements[0] > kMaxElements)
        return fail(HYLE_HIP_UNIMPLEMENTED, "Softmax requires at most INT32_MAX elements");
      if (same_desc(in[0], out)) p->alias_inputs[0] = 1;
      if (p->output_elements[0] == 0) return HYLE_HIP_OK;
      int axis;
      if ((s = normalize_axis(r.axis, in[0].rank, &axis)) != HYLE_HIP_OK) return s;
      p->route = Route::kSoftmax;
      p->dispatches = 1;
      const int rank = in[0].rank;
      const uint32_t width = (uint32_t)in[0].dims[axis];
      // general description (any axis, any strides)
      SoftmaxGeneralParams &g = p->softmax_general;
      g.width = width;
      g.scale = r.scale;
      g.mask_kind = (uint8_t)r.mask;
      g.log = r.kind2 == HYLE_HIP_LOG_SOFTMAX;
      g.rank = rank;
      g.axis = axis;
      g.outer = g.inner = 1;
      for (int a = 0; a < rank; ++a) {
        g.dims[a] = (uint32_t)in[0].dims[a];
        g.in_strides[a] = in[0].byte_strides[a];
        if (a < axis) g.outer *= (uint64_t)in[0].dims[a];
        if (a > axis) g.inner *= (uint64_t)in[0].dims[a];
      }
      if (r.mask != HYLE_HIP_MASK_NONE) {
        for (int rev = 0; rev < rank; ++rev) {
          const int a = rank - 1 - rev;
          int64_t stride = 0;
          if (rev < in[1].rank) {
            const int ma = in[1].rank - 1 - rev;
            if (in[1].dims[ma] != 1) stride = in[1].byte_strides[ma];
          }
          g.mask_strides[a] = stride;
        }
      }
      // row kernel: dense input, last axis
      p->softmax_rows_ok = axis == rank - 1 && is_dense(in[0]);
      if (p->softmax_rows_ok) {
        SoftmaxParams &sp = p->softmax;
        sp.shape.width = width;
        sp.shape.rows = p->output_elements[0] / width;
        sp.scale = r.scale;
        sp.mask_kind = (uint8_t)r.mask;
        sp.log = g.log;
        sp.outer_rank = rank - 1;
        for (int a = 0; a < rank - 1; ++a) {
          sp.outer_dims[a] = g.dims[a];
          sp.mask_outer_strides[a] = g.mask_strides[a];
        }
        sp.mask_inner_stride = g.mask_strides[rank - 1];
        p->softmax_mask_vector_ok = true;
        if (r.mask != HYLE_HIP_MASK_NONE) {
          const int64_t unit = (int64_t)dtype_size(in[1].dtype);
          if (sp.mask_inner_stride != 0 && sp.mask_inner_stride != unit)
            p->softmax_mask_vector_ok = false;
          // a mask row is read as whole vectors: one byte per column for Bool, one
          // element per column for an additive mask
          const int64_t row_alignment = r.mask == HYLE_HIP_MASK_BOOLEAN ? elem_vec(p->elem) : 16;
          for (int a = 0; a < rank - 1; ++a)
            if (sp.mask_outer_strides[a] % row_alignment != 0) p->softmax_mask_vector_ok = false;
        }
      }
      return HYLE_HIP_OK;
    }
    case HYLE_HIP_OP_REDUCE: {
      // src/compute_provider_cuda/reduction_provider.cc:40-107: plain f32/f16/bf16 with any
      // byte strides, dense output, f32 accumulation (explicit for the narrow types), at most
      // INT32_MAX elements on either side; an empty reduced extent still writes identities.
      if (!to_elem(in[0].dtype, &p->elem) || !is_plain(in[0]))
        return fail(HYLE_HIP_UNIMPLEMENTED, "Reduce requires plain float32/float16/bfloat16");
      if ((s = require_f32_accumulation(p, in[0].dtype, "Reduce")) != HYLE_HIP_OK) return s;
      uint32_t selected;
      if ((s = reduce_axes(r, in[0].rank, &selected)) != HYLE_HIP_OK) return s;
      if (p->input_elements[0] > kMaxElements || p->output_elements[0] > kMaxElements)
        return fail(HYLE_HIP_UNIMPLEMENTED, "Reduce requires at most INT32_MAX elements");
      if (p->output_elements[0] == 0) return HYLE_HIP_OK;
      ReduceParams &rp = p->reduce;
      rp = ReduceParams{};
      rp.kind = (uint8_t)r.kind;
      rp.rows = (uint32_t)p->output_elements[0];
      rp.width = (uint32_t)(p->input_elements[0] / p->output_elements[0]);
      rp.divisor = (float)rp.width;
      const int64_t size = (int64_t)dtype_size(in[0].dtype);
      // Runs of neighbouring axes with the same fate (extent-1 axes belong to either run).
      int groups = 0;
      bool group_reduced[HYLE_HIP_MAX_RANK];
      uint64_t group_extent[HYLE_HIP_MAX_RANK];
      for (int a = 0; a < in[0].rank; ++a) {
        if (in[0].dims[a] == 1) continue;
        const bool reduced = ((selected >> a) & 1u) != 0;
        if (groups != 0 && group_reduced[groups - 1] == reduced) {
          group_extent[groups - 1] *= (uint64_t)in[0].dims[a];
        } else {
          group_reduced[groups] = reduced;
          group_extent[groups++] = (uint64_t)in[0].dims[a];
        }
      }
      const bool dense = is_dense(in[0]) || rp.width == 0;
      if (dense && (groups == 0 || rp.width == 0 || (groups == 1 && group_reduced[0]) ||
                    (groups == 2 && !group_reduced[0]))) {
        rp.form = ReduceForm::kRows;  // "", "R", "KR"
      } else if (dense && ((groups == 1 && !group_reduced[0]) || (groups == 2 && group_reduced[0]) ||
                           (groups == 3 && !group_reduced[0]))) {
        rp.form = ReduceForm::kColumns;  // "K" (nothing to fold), "RK", "KRK"
        rp.inner = (uint32_t)group_extent[groups - 1];
        rp.reduced = groups == 1 ? 1u : (uint32_t)group_extent[groups - 2];
        rp.outer = groups == 3 ? (uint32_t)group_extent[0] : 1u;
      } else {
        rp.form = ReduceForm::kGeneral;
        rp.rank = in[0].rank;
        rp.axes = selected;
        for (int a = 0; a < in[0].rank; ++a) {
          rp.dims[a] = (uint32_t)in[0].dims[a];
          rp.strides[a] = in[0].byte_strides[a];
          if (in[0].dims[a] > 1 && in[0].byte_strides[a] % size != 0) rp.bytewise = true;
        }
        if (rp.bytewise) p->input_alignment[0] = 1;
      }
      reduce_plan(p->elem, &rp);
      p->route = Route::kReduce;
      p->dispatches = rp.dispatches;
      p->workspace_size = rp.workspace_bytes;
      p->workspace_alignment = rp.workspace_bytes != 0 ? 16 : 1;
      return HYLE_HIP_OK;
    }
    case HYLE_HIP_OP_TOP_K: {
      // include/hyle/compute/providers/cuda.h:113-117: plain rank <= 8 byte strides, dense
      // outputs, no aliases, caller-owned workspace.
      const bool integer = in[0].dtype == HYLE_HIP_DTYPE_I32;
      if ((!integer && !to_elem(in[0].dtype, &p->elem)) || !is_plain(in[0]))
        return fail(HYLE_HIP_UNIMPLEMENTED, "TopK requires plain float32/float16/bfloat16/int32");
      int axis;
      if ((s = normalize_axis(r.axis, in[0].rank, &axis)) != HYLE_HIP_OK) return s;
      if (p->input_elements[0] > kMaxElements)
        return fail(HYLE_HIP_UNIMPLEMENTED, "TopK requires at most INT32_MAX elements");
      if (p->output_elements[0] == 0) return HYLE_HIP_OK;
      bool innermost = is_dense(in[0]);  // dense, and nothing but extent-1 axes after the axis
      for (int a = axis + 1; a < in[0].rank; ++a)
        if (in[0].dims[a] != 1) innermost = false;
      if (r.count == 1 && r.largest && innermost && !integer) {
        // the vocabulary argmax: a scan dispatch and a fold dispatch
        p->route = Route::kArgmax;
        argmax_plan(p->output_elements[0], (uint32_t)in[0].dims[axis], p->elem, units, &p->argmax);
        p->workspace_size = argmax_workspace_bytes(p->argmax);
        p->workspace_alignment = 16;
        p->dispatches = 2;
        return HYLE_HIP_OK;
      }
      TopKParams &t = p->topk;
      t = TopKParams{};
      t.integer = integer;
      t.count = (uint32_t)r.count;
      t.rows = (uint32_t)(p->output_elements[0] / r.count);
      t.width = (uint32_t)in[0].dims[axis];
      t.largest = r.largest != 0;
      t.dense_last = innermost;
      t.rank = in[0].rank;
      t.axis = axis;
      const int64_t size = (int64_t)dtype_size(in[0].dtype);
      for (int a = 0; a < in[0].rank; ++a) {
        t.dims[a] = (uint32_t)in[0].dims[a];
        t.strides[a] = in[0].byte_strides[a];
        if (a > axis) t.inner *= (uint32_t)in[0].dims[a];
        if (in[0].dims[a] > 1 && in[0].byte_strides[a] % size != 0) t.bytewise = true;
      }
      if (t.bytewise) p->input_alignment[0] = 1;
      topk_plan(&t);
      p->route = Route::kTopK;
      p->dispatches = t.dispatches;
      p->workspace_size = t.workspace_bytes;
      p->workspace_alignment = t.workspace_bytes != 0 ? 16 : 1;
      return HYLE_HIP_OK;
    }
    case HYLE_HIP_OP_Q8_0_DEQUANT_SUMSQ: {
      const int64_t k = in[0].dims[0], n = in[0].dims[1];
      const int64_t per_block = in[0].elements_per_block, block_bytes = in[0].bytes_per_block;
      if ((s = admit_gguf_rows(in[0])) != HYLE_HIP_OK) return s;
      p->elem = Elem::kBF16;
      if (n == 0) return HYLE_HIP_OK;
      if (per_block == 256) {
        // Q4_K / Q6_K: the blocks are read at any byte address; the bf16 rows are stored as
        // 16-byte vectors
        p->route = Route::kKQuantDequant;
        p->kquant.rows = (uint64_t)n;
        p->kquant.k = (uint32_t)k;
        p->kquant.row_stride = (uint64_t)in[0].byte_strides[1];
        p->kquant.kind = block_bytes == 144 ? 0 : 1;
        p->input_alignment[0] = 1;
        p->output_alignment[0] = 16;
        p->dispatches = 1;
        return HYLE_HIP_OK;
      }
      // with K == 0 the bf16 output is empty but every row still gets sumsq = 0
      p->route = Route::kQ8Dequant;
      p->q8.rows = (uint64_t)n;
      p->q8.k = (uint32_t)k;
      p->q8.row_stride = (uint64_t)in[0].byte_strides[1];
      p->dispatches = 1;
      return HYLE_HIP_OK;
    }
    case HYLE_HIP_OP_GGUF_MATVEC: {
      const int64_t k = in[0].dims[0], n = in[0].dims[1];
      const int64_t per_block = in[0].elements_per_block, block_bytes = in[0].bytes_per_block;
      if (!to_elem(in[1].dtype, &p->elem) || !is_plain(in[1]) || !is_dense(in[1]))
        return fail(HYLE_HIP_UNIMPLEMENTED, "GGUF matvec requires dense plain float32/float16/bfloat16 activations");
      if ((s = admit_gguf_rows(in[0])) != HYLE_HIP_OK) return s;
      const int64_t m = in[1].rank == 2 ? in[1].dims[0] : 1;
      if (m > 8) return fail(HYLE_HIP_UNIMPLEMENTED, "GGUF matvec serves at most 8 activation rows");
      const uint8_t matvec_kind = per_block == 32 ? 2 : (block_bytes == 144 ? 0 : 1);
      if (r.kind2 == HYLE_HIP_ACTIVATIONS_GGML_Q8) {
        // any whole number of blocks per row; the blocks are read as 16-bit aligned pieces, so rows
        // start at even addresses; one activation row's 8-bit codes must fit a block's LDS
        if (in[0].byte_strides[1] % 2 != 0)
          return fail(HYLE_HIP_UNIMPLEMENTED, "GGUF matvec with 8-bit activation blocks serves rows at even byte strides");
        if (!gguf_matvec_q8_serves(matvec_kind, (uint32_t)k))
          return fail(HYLE_HIP_UNIMPLEMENTED, "GGUF matvec keeps the activation codes in LDS: K is too large");
        p->input_alignment[0] = 2;
      } else if (gguf_matvec_shared_bytes((uint32_t)m, (uint32_t)k) > 64 * 1024) {
        return fail(HYLE_HIP_UNIMPLEMENTED, "GGUF matvec keeps the activations in LDS: M * K is too large");
      }
      if (p->output_elements[0] == 0) return HYLE_HIP_OK;
      p->route = Route::kGgufMatVec;
      p->matvec.codec = (uint8_t)r.kind2;
      p->matvec.compute_units = units;
      p->matvec.rows = (uint64_t)n;
      p->matvec.k = (uint32_t)k;
      p->matvec.m = (uint32_t)m;
      p->matvec.row_stride = (uint64_t)in[0].byte_strides[1];
      p->matvec.kind = matvec_kind;
      if (r.kind2 != HYLE_HIP_ACTIVATIONS_GGML_Q8) p->input_alignment[0] = 1;
      p->dispatches = r.kind2 == HYLE_HIP_ACTIVATIONS_GGML_Q8
                          ? gguf_matvec_q8_dispatches(matvec_kind, (uint32_t)m, (uint32_t)k, (uint64_t)in[0].byte_strides[1])
                          : 1;
      return HYLE_HIP_OK;
    }
    case HYLE_HIP_OP_FILL: {
      // storage only: the scalar's bits go to every element (src/compute_provider_cuda/
      // tensor_provider.cc:85-98, tensor_kernel.cu:190-193)
      const uint64_t n = p->output_elements[0];
      if (n > kMaxElements) return fail(HYLE_HIP_UNIMPLEMENTED, "Fill output exceeds INT32_MAX elements");
      if (n == 0) return HYLE_HIP_OK;
      const size_t size = dtype_size(out.dtype);
      if (size < 8 && (r.count >> (8 * size)) != 0)
        return fail(HYLE_HIP_INVALID_ARGUMENT, "Fill scalar bits do not fit the output type");
      p->route = Route::kFill;
      p->dispatches = 1;
      p->fill.elements = n;
      p->fill.bits = r.count;
      p->fill.size = (uint8_t)size;
      return HYLE_HIP_OK;
    }
    case HYLE_HIP_OP_SELECT: {
      // storage only, plain operands broadcast to a dense output (src/compute_provider_cuda/
      // tensor_provider.cc:85-90,119-121,176-195; tensor_kernel.cu:194-198)
      for (int i = 0; i < 3; ++i)
        if (!is_plain(in[i])) return fail(HYLE_HIP_UNIMPLEMENTED, "Select requires plain storage");
      const uint64_t n = p->output_elements[0];
      if (n > kMaxElements) return fail(HYLE_HIP_UNIMPLEMENTED, "Select output exceeds INT32_MAX elements");
      if (n == 0) return HYLE_HIP_OK;
      // a branch whose descriptor is the output's may be written in place; the condition may not
      for (int i = 1; i < 3; ++i)
        if (same_desc(in[i], out)) p->alias_inputs[0] |= (uint8_t)(1u << i);
      SelectParams &sel = p->select;
      sel.elements = n;
      sel.size = (uint8_t)dtype_size(out.dtype);
      sel.flat = true;
      for (int i = 0; i < 3; ++i) {
        uint32_t period = 0;
        sel.flat = sel.flat && suffix_period(in[i], out, n, &period) && period <= 1;
        sel.scalar[i] = period == 1;
      }
      sel.rank = out.rank;
      for (int a = 0; a < out.rank; ++a) sel.dims[a] = (uint32_t)out.dims[a];
      for (int i = 0; i < 3; ++i) {
        for (int rev = 0; rev < out.rank; ++rev) {
          int64_t stride = 0;
          if (rev < in[i].rank && in[i].dims[in[i].rank - 1 - rev] != 1) stride = in[i].byte_strides[in[i].rank - 1 - rev];
          sel.strides[i][out.rank - 1 - rev] = stride;
        }
        // the strided kernel gathers bytes, so byte strides need not keep elements aligned
        if (!sel.flat) p->input_alignment[i] = 1;
      }
      p->route = Route::kSelect;
      p->dispatches = 1;
      return HYLE_HIP_OK;
    }
    case HYLE_HIP_OP_CONCAT: {
      // src/compute_provider_cuda/concat_provider.cc:40-90
      for (uint32_t i = 0; i < r.input_count; ++i)
        if (!is_plain(in[i])) return fail(HYLE_HIP_UNIMPLEMENTED, "Concat requires plain inputs and a dense output");
      const uint64_t n = p->output_elements[0];
      if (n > kMaxElements) return fail(HYLE_HIP_UNIMPLEMENTED, "Concat output exceeds INT32_MAX elements");
      if (n == 0) return HYLE_HIP_OK;
      int axis = 0;
      normalize_axis(r.axis, out.rank, &axis);
      ConcatParams &c = p->concat;
      c.elements = n;
      c.inputs = r.input_count;
      c.size = (uint8_t)dtype_size(out.dtype);
      c.rank = out.rank;
      c.axis = axis;
      c.total = (uint32_t)out.dims[axis];
      c.outer = c.inner = 1;
      for (int a = 0; a < out.rank; ++a) {
        c.dims[a] = (uint32_t)out.dims[a];
        if (a < axis) c.outer *= (uint32_t)out.dims[a];
        if (a > axis) c.inner *= (uint32_t)out.dims[a];
      }
      uint32_t start = (uint32_t)r.count;
      c.dense = true;
      bool any = false;
      for (uint32_t i = 0; i < r.input_count; ++i) {
        c.extent[i] = (uint32_t)in[i].dims[axis];
        c.offset[i] = start;
        start += c.extent[i];
        any = any || p->input_elements[i] != 0;
        if (p->input_elements[i] == 0) continue;
        c.dense = c.dense && is_dense(in[i]);
        uint64_t last = 0;  // byte offset of the last element: TensorDesc::required_bytes
        for (int a = 0; a < in[i].rank; ++a) {
          c.strides[i][a] = in[i].byte_strides[a];
          last += (uint64_t)(in[i].dims[a] - 1) * (uint64_t)in[i].byte_strides[a];
        }
        p->concat_input_bytes[i] = last + c.size;
      }
      if (!any) return HYLE_HIP_OK;  // an empty group: nothing to dispatch, no pointer is touched
      if (!c.dense)
        for (uint32_t i = 0; i < r.input_count; ++i) p->input_alignment[i] = 1;  // gathered bytewise
      p->route = Route::kConcat;
      p->dispatches = 1;
      return HYLE_HIP_OK;
    }
    case HYLE_HIP_OP_ROPE: {
      // the reference's explicit-frequency route takes dense operands and f32 frequencies
      // (src/compute_ggml_runtime/explicit_rope.h:11-40)
      if (!to_elem(in[0].dtype, &p->elem) || !is_dense(in[0]) || !is_plain(in[0]))
        return fail(HYLE_HIP_UNIMPLEMENTED, "RoPE requires dense float32/float16/bfloat16 data");
      if (!is_plain(in[1]) || !is_dense(in[1]) || !is_plain(in[2]) || !is_dense(in[2]) || in[2].dtype != HYLE_HIP_DTYPE_F32)
        return fail(HYLE_HIP_UNIMPLEMENTED, "RoPE requires dense positions and dense float32 frequencies");
      const uint64_t n = p->output_elements[0];
      if (n > kMaxElements) return fail(HYLE_HIP_UNIMPLEMENTED, "RoPE requires at most INT32_MAX elements");
      p->alias_inputs[0] = 1;  // a thread reads both elements of its pairs before it writes them
      if (n == 0) return HYLE_HIP_OK;
      int sequence_axis = 0;
      normalize_axis(r.axis, in[0].rank, &sequence_axis);
      RopeParams &rope = p->rope;
      rope.depth = (uint32_t)in[0].dims[in[0].rank - 1];
      rope.rows = n / rope.depth;
      rope.rotary = (uint32_t)r.count;
      rope.sequence = (uint32_t)in[0].dims[sequence_axis];
      rope.inner = 1;
      for (int a = sequence_axis + 1; a < in[0].rank - 1; ++a) rope.inner *= (uint32_t)in[0].dims[a];
      rope.half_split = r.kind2 == HYLE_HIP_ROPE_HALF_SPLIT;
      rope.wide_positions = in[1].dtype == HYLE_HIP_DTYPE_I64;
      rope.batched_positions = in[1].rank > 1;
      rope.stepped_frequencies = in[2].rank == 2;
      p->route = Route::kRope;
      p->dispatches = 1;
      return HYLE_HIP_OK;
    }
    case HYLE_HIP_OP_RANDOM_BITS: {
      // src/compute_provider_cuda/sampling_provider.cc:26-71
      if (p->input_elements[0] / 4 > kMaxElements || p->output_elements[0] > kMaxElements)
        return fail(HYLE_HIP_UNIMPLEMENTED, "RandomBits requires at most INT32_MAX rows and output words");
      if (p->output_elements[0] == 0) return HYLE_HIP_OK;
      p->route = Route::kRandomBits;
      p->dispatches = 1;
      p->random_bits.rows = (uint32_t)in[0].dims[0];
      p->random_bits.word_count = (uint32_t)r.count;
      return HYLE_HIP_OK;
    }
    case HYLE_HIP_OP_CATEGORICAL: {
      // src/compute_provider_cuda/sampling_provider.cc:26-71: fixed shapes, row and tile grids within I32
      if (!to_elem(in[0].dtype, &p->elem)) return fail(HYLE_HIP_UNIMPLEMENTED, "Categorical requires float32/float16/bfloat16");
      const uint64_t rows = (uint64_t)in[0].dims[0], width = (uint64_t)in[0].dims[1];
      const uint64_t tiles = (width + kCategoricalTile - 1) / kCategoricalTile;
      if (rows > kMaxElements || rows * tiles > kMaxElements)
        return fail(HYLE_HIP_UNIMPLEMENTED, "Categorical row or tile grid capacity exceeded");
      if (rows == 0) return HYLE_HIP_OK;
      CategoricalParams &c = p->categorical;
      c.rows = (uint32_t)rows;
      c.width = (uint32_t)width;
      c.tiles = (uint32_t)tiles;
      c.scored = r.kind2 == 1;
      c.status_offset = (rows * tiles * sizeof(CategoricalTile) + 255) / 256 * 256;
      p->workspace_size = c.status_offset + 256;
      p->workspace_alignment = 256;
      p->route = Route::kCategorical;
      p->dispatches = 2;
      return HYLE_HIP_OK;
    }
    case HYLE_HIP_OP_GATHER: {
      // src/compute_provider_cuda/collectives_provider.cc:92-125: plain source and indices, at
      // most INT32_MAX output elements and indices
      if (!is_plain(in[0]) || !is_plain(in[1]) || in[0].rank == 0)
        return fail(HYLE_HIP_UNIMPLEMENTED, "Gather requires a plain source of rank >= 1 and plain indices");
      const uint64_t n = p->output_elements[0];
      if (n > kMaxElements || p->input_elements[1] > kMaxElements)
        return fail(HYLE_HIP_UNIMPLEMENTED, "Gather output or index count exceeds INT32_MAX");
      if (n == 0) return HYLE_HIP_OK;
      int axis = 0;
      normalize_axis(r.axis, in[0].rank, &axis);
      GatherParams &g = p->gather;
      const int64_t size = (int64_t)dtype_size(out.dtype);
      g.elements = n;
      g.size = (uint8_t)size;
      g.extent = (uint64_t)in[0].dims[axis];
      g.wide_indices = in[1].dtype == HYLE_HIP_DTYPE_I64;
      g.dense_indices = is_dense(in[1]);
      g.checked = r.kind2 == HYLE_HIP_BOUNDS_CHECKED;
      g.index_count = (uint32_t)p->input_elements[1];
      g.index_rank = in[1].rank;
      for (int a = 0; a < in[1].rank; ++a) {
        g.index_dims[a] = (uint32_t)in[1].dims[a];
        g.index_strides[a] = in[1].dims[a] == 1 ? 0 : in[1].byte_strides[a];
      }
      g.axis_pitch = (uint64_t)in[0].byte_strides[axis];
      g.outer = 1;
      g.inner = 1;
      for (int a = 0; a < axis; ++a) g.outer *= (uint32_t)in[0].dims[a];
      for (int a = axis + 1; a < in[0].rank; ++a) g.inner *= (uint64_t)in[0].dims[a];
      // whole rows move when the elements after the axis are contiguous and the axes before it
      // fold into one pitch (axes of extent 1 have no say)
      g.rows = true;
      int64_t expected = size;
      for (int a = in[0].rank - 1; a > axis; --a) {
        if (in[0].dims[a] != 1 && in[0].byte_strides[a] != expected) g.rows = false;
        expected *= in[0].dims[a];
      }
      bool first = true;
      expected = 0;
      for (int a = axis - 1; a >= 0; --a) {
        if (in[0].dims[a] == 1) continue;
        if (first) g.outer_pitch = (uint64_t)in[0].byte_strides[a];
        else if (in[0].byte_strides[a] != expected) g.rows = false;
        first = false;
        expected = in[0].byte_strides[a] * in[0].dims[a];
      }
      // the coordinate walk: per output axis, the source's stride or the indices'
      g.rank = out.rank;
      for (int a = 0; a < out.rank; ++a) {
        g.dims[a] = (uint32_t)out.dims[a];
        if (a < axis) g.source_strides[a] = in[0].byte_strides[a];
        else if (a < axis + in[1].rank) g.index_out_strides[a] = g.index_strides[a - axis];
        else g.source_strides[a] = in[0].byte_strides[a - in[1].rank + 1];
      }
      // strided operands may sit at any byte: they are read bytewise
      if (!is_dense(in[0])) p->input_alignment[0] = 1;
      if (!g.dense_indices) p->input_alignment[1] = 1;
      for (int i = 0; i < 2; ++i) {
        uint64_t last = 0;  // byte offset of the last element: TensorDesc::required_bytes
        for (int a = 0; a < in[i].rank; ++a) last += (uint64_t)(in[i].dims[a] - 1) * (uint64_t)in[i].byte_strides[a];
        p->concat_input_bytes[i] = p->input_elements[i] == 0 ? 0 : last + dtype_size(in[i].dtype);
      }
      // Few indices (the rows a step picks for its last tokens, a decode batch's embeddings): every
      // moving block looks at all of them itself, which saves the checking dispatch.  At most 1024
      // indices, and at most 8 MiB of index reads over all blocks, counted for the narrowest units.
      // Long rows in a launch large enough for the blocks of sixteen chunks (4096 chunks of 4 KiB,
      // whatever unit the addresses allow) check while their rows are on the way, which hides the
      // index reads: up to 16384 indices and 32 MiB of index reads, counted for 16-byte units
      // (8192 checked rows of 4 KiB: 12.4 us in one dispatch against 14.5 us in two).
      const uint64_t index_bytes = (uint64_t)g.index_count * (g.wide_indices ? 8 : 4);
      const uint64_t row_bytes = g.inner * (uint64_t)size, row_count = (uint64_t)g.outer * g.index_count;
      const uint64_t chunks = (row_bytes + 4095) / 4096 * row_count;
      const bool few = g.index_count <= 1024 && (n + 255) / 256 * index_bytes <= (8u << 20);
      const bool overlapped = row_bytes >= 4096 && chunks >= 4096 && g.index_count <= 16384 &&
                              (chunks + 15) / 16 * index_bytes <= (32u << 20);
      g.fused_check = g.checked && g.rows && (few || overlapped);
      p->route = Route::kGather;
      p->dispatches = g.checked && !g.fused_check ? 2 : 1;
      if (g.checked) {
        p->workspace_size = kGatherWorkspaceBytes;
        p->workspace_alignment = 256;
      }
      return HYLE_HIP_OK;
    }
    case HYLE_HIP_OP_COPY:
    case HYLE_HIP_OP_CAST: {
      // src/compute_provider_native/cast.cc:127-176,256-279 (admitted pairs, plain input, dense
      // output) and transform.cc:171-179 (Copy of plain storage).
      CastParams &c = p->cast;
      auto cast_type = [](uint8_t dtype, CastType *t) {
        switch (dtype) {
          case HYLE_HIP_DTYPE_F32: *t = CastType::kF32; return true;
          case HYLE_HIP_DTYPE_F16: *t = CastType::kF16; return true;
          case HYLE_HIP_DTYPE_BF16: *t = CastType::kBF16; return true;
          case HYLE_HIP_DTYPE_BOOL: *t = CastType::kBool; return true;
          case HYLE_HIP_DTYPE_I32: *t = CastType::kI32; return true;
          default: return false;
        }
      };
      if (in[0].dtype == out.dtype) {
        c.copy_size = (uint8_t)dtype_size(out.dtype);  // equal types keep the bytes
      } else {
        const bool pair_ok = cast_type(in[0].dtype, &c.src) && cast_type(out.dtype, &c.dst) &&
                             ((is_floating(in[0].dtype) && is_floating(out.dtype)) ||
                              (in[0].dtype == HYLE_HIP_DTYPE_I32 && out.dtype == HYLE_HIP_DTYPE_F32) ||
                              (in[0].dtype == HYLE_HIP_DTYPE_BOOL && is_floating(out.dtype)) ||
                              (is_floating(in[0].dtype) && out.dtype == HYLE_HIP_DTYPE_BOOL));
        if (!pair_ok)
          return fail(HYLE_HIP_UNIMPLEMENTED, "Cast storage conversion pair is not admitted");
      }
      const uint64_t n = p->output_elements[0];
      if (n > kMaxElements)
        return fail(HYLE_HIP_UNIMPLEMENTED, "Cast / Copy output exceeds INT32_MAX elements");
      if (n == 0) return HYLE_HIP_OK;
      c.elements = n;
      c.dense_input = is_dense(in[0]);
      c.rank = in[0].rank;
      uint64_t last = 0;  // byte offset of the last element: TensorDesc::required_bytes
      for (int a = 0; a < in[0].rank; ++a) {
        c.dims[a] = (uint32_t)in[0].dims[a];
        c.strides[a] = in[0].byte_strides[a];
        last += (uint64_t)(in[0].dims[a] - 1) * (uint64_t)in[0].byte_strides[a];
      }
      if (c.copy_size == 8) {
        // an 8-byte element moves as two 4-byte halves: one more innermost axis of extent 2
        if (2 * n > kMaxElements || (!c.dense_input && c.rank == kMaxRank))
          return fail(HYLE_HIP_UNIMPLEMENTED, "Copy of 8-byte elements exceeds INT32_MAX halves or rank 7 with strides");
        c.copy_size = 4;
        c.elements = 2 * n;
        c.dims[c.rank] = 2;
        c.strides[c.rank] = 4;
        c.rank += 1;
      }
      p->route = Route::kCast;
      p->dispatches = 1;
      // byte strides need not keep elements aligned (cast.cc:113-116): such inputs are read bytewise
      if (!c.dense_input) p->input_alignment[0] = 1;
      p->no_overlap_input_bytes = last + dtype_size(in[0].dtype);
      p->no_overlap_output_bytes = n * dtype_size(out.dtype);
      return HYLE_HIP_OK;
    }
    default:
      return fail(HYLE_HIP_UNIMPLEMENTED, "operation kind %u is not served by this provider", r.op);
  }
}

bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

}  // namespace

namespace hyle_hip {
namespace variants {
const char *add(const std::string &label) {
  VariantList &list = variant_list();
  std::lock_guard<std::mutex> lock(list.mutex);
  for (const std::string *known : list.labels)
    if (*known == label) return known->c_str();
  list.labels.push_back(new std::string(label));
  return list.labels.back()->c_str();
}
void note(const char *label) {
  // a loop of dispatches of one shape (merge rounds) is one entry
  if (g_noted_count != 0 && g_noted[g_noted_count - 1] == label) return;
  if (g_noted_count < kNotedVariants) g_noted[g_noted_count++] = label;
}
}  // namespace variants
}  // namespace hyle_hip

// ---------------------------------------------------------------------------------
// Device scratch of hyle_hip_plan_launch_static: the workspace of the two-dispatch routes for
// callers that cannot allocate.  Every device the library runs on holds its own copy of the
// array at its own address until the process ends.  In host code the array's name is only a
// stand-in for the symbol, never a device address: the address is looked up once per device,
// with that device current, and only that pointer is handed to kernels.
// ---------------------------------------------------------------------------------
constexpr size_t kStaticScratchBytes = HYLE_HIP_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_address[kMaxDevices] = {};

// The address of `scratch` on `device`, resolved on first use.  The calling thread's current
// device is left as it was.
hyle_hip_status static_scratch_address(int device, void **address) {
  *address = nullptr;
  if (device < 0 || device >= kMaxDevices)
    return fail(HYLE_HIP_INVALID_ARGUMENT, "device %d is outside the %d devices the scratch table holds", device,
                kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_address[device] == nullptr) {
    int previous = 0;
    hipError_t err = hipGetDevice(&previous);
    if (err != hipSuccess) return hip_fail(err, "hipGetDevice");
    if (previous != device && (err = hipSetDevice(device)) != hipSuccess) return hip_fail(err, "hipSetDevice");
    void *found = nullptr;
    err = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
    if (previous != device) (void)hipSetDevice(previous);
    if (err != hipSuccess) return hip_fail(err, "hipGetSymbolAddress(scratch)");
    if (found == nullptr || !aligned(found, 256))
      return fail(HYLE_HIP_INTERNAL, "device scratch has no usable address on device %d", device);
    g_scratch_address[device] = found;
  }
  *address = g_scratch_address[device];
  return HYLE_HIP_OK;
}

}  // namespace

// ---------------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------------
extern "C" {

uint32_t hyle_hip_abi_version(void) { return HYLE_HIP_ABI_VERSION; }

const char *hyle_hip_last_error(void) { return g_error; }

const char *hyle_hip_status_name(hyle_hip_status status) {
  switch (status) {
    case HYLE_HIP_OK: return "OK";
    case HYLE_HIP_CANCELLED: return "CANCELLED";
    case HYLE_HIP_INVALID_ARGUMENT: return "INVALID_ARGUMENT";
    case HYLE_HIP_RESOURCE_EXHAUSTED: return "RESOURCE_EXHAUSTED";
    case HYLE_HIP_FAILED_PRECONDITION: return "FAILED_PRECONDITION";
    case HYLE_HIP_OUT_OF_RANGE: return "OUT_OF_RANGE";
    case HYLE_HIP_UNIMPLEMENTED: return "UNIMPLEMENTED";
    case HYLE_HIP_INTERNAL: return "INTERNAL";
    case HYLE_HIP_UNAVAILABLE: return "UNAVAILABLE";
  }
  return "UNKNOWN";
}

hyle_hip_status hyle_hip_context_create(int device, hyle_hip_context **context) {
  if (context == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "context output is null");
  *context = nullptr;
  int count = 0;
  hipError_t err = hipGetDeviceCount(&count);
  if (err != hipSuccess || count <= 0) {
    (void)hipGetLastError();
    return fail(HYLE_HIP_UNAVAILABLE, "no HIP device is visible");
  }
  if (device < 0 || device >= count)
    return fail(HYLE_HIP_INVALID_ARGUMENT, "device %d is outside [0, %d)", device, count);
  hipDeviceProp_t props;
  err = hipGetDeviceProperties(&props, device);
  if (err != hipSuccess) return hip_fail(err, "hipGetDeviceProperties");
  if (std::strncmp(props.gcnArchName, "gfx950", 6) != 0)
    return fail(HYLE_HIP_UNAVAILABLE, "device %d is %s; this provider carries gfx950 code only", device,
                props.gcnArchName);
  auto *ctx = new (std::nothrow) hyle_hip_context;
  if (ctx == nullptr) return fail(HYLE_HIP_RESOURCE_EXHAUSTED, "out of host memory");
  ctx->device = device;
  ctx->compute_units = props.multiProcessorCount;
  const hyle_hip_status scratch_status = static_scratch_address(device, &ctx->static_scratch);
  if (scratch_status != HYLE_HIP_OK) {
    delete ctx;
    return scratch_status;
  }
  *context = ctx;
  return HYLE_HIP_OK;
}

void hyle_hip_context_destroy(hyle_hip_context *context) { delete context; }

int hyle_hip_context_compute_units(const hyle_hip_context *context) {
  return context ? context->compute_units : 0;
}

hyle_hip_status hyle_hip_infer_outputs(const hyle_hip_op_desc *request, hyle_hip_tensor_desc *outputs,
                                       uint32_t *output_count) {
  if (request == nullptr || outputs == nullptr || output_count == nullptr)
    return fail(HYLE_HIP_INVALID_ARGUMENT, "null argument");
  Desc local[HYLE_HIP_MAX_OUTPUTS];
  uint32_t count = 0;
  hyle_hip_status s = infer(*request, local, &count);
  if (s != HYLE_HIP_OK) return s;
  for (uint32_t i = 0; i < count; ++i) outputs[i] = local[i];
  *output_count = count;
  return HYLE_HIP_OK;
}

hyle_hip_status hyle_hip_plan_create(hyle_hip_context *context, const hyle_hip_op_desc *request,
                                     const hyle_hip_tensor_desc *outputs, uint32_t output_count,
                                     hyle_hip_plan **plan) {
  if (plan == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "plan output is null");
  *plan = nullptr;
  if (request == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "request is null");
  auto *p = new (std::nothrow) hyle_hip_plan;
  if (p == nullptr) return fail(HYLE_HIP_RESOURCE_EXHAUSTED, "out of host memory");
  p->context = context;
  p->request = *request;
  hyle_hip_status s = infer(p->request, p->outputs, &p->output_count);
  if (s == HYLE_HIP_OK && outputs != nullptr) {
    if (output_count != p->output_count)
      s = fail(HYLE_HIP_INVALID_ARGUMENT, "operation output span must have the exact output count");
    for (uint32_t i = 0; s == HYLE_HIP_OK && i < output_count; ++i)
      if (!same_desc(outputs[i], p->outputs[i]))
        s = fail(HYLE_HIP_INVALID_ARGUMENT,
                 "output %u descriptor differs from the inferred dense description", i);
  }
  if (s == HYLE_HIP_OK) {
    for (uint32_t i = 0; i < p->request.input_count; ++i) {
      element_count(p->request.inputs[i], &p->input_elements[i]);
      p->input_alignment[i] =
          is_plain(p->request.inputs[i]) ? dtype_size(p->request.inputs[i].dtype) : 1;
    }
    for (uint32_t i = 0; i < p->output_count; ++i) {
      element_count(p->outputs[i], &p->output_elements[i]);
      p->output_alignment[i] = dtype_size(p->outputs[i].dtype);
    }
    s = admit(p);
  }
  if (s != HYLE_HIP_OK) {
    delete p;
    return s;
  }
  *plan = p;
  return HYLE_HIP_OK;
}

void hyle_hip_plan_destroy(hyle_hip_plan *plan) { delete plan; }

hyle_hip_status hyle_hip_plan_workspace(const hyle_hip_plan *plan, size_t *size, size_t *alignment) {
  if (plan == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "plan is null");
  if (size) *size = plan->workspace_size;
  if (alignment) *alignment = plan->workspace_alignment;
  return HYLE_HIP_OK;
}

hyle_hip_status hyle_hip_plan_outputs(const hyle_hip_plan *plan, hyle_hip_tensor_desc *outputs,
                                      uint32_t *output_count) {
  if (plan == nullptr || outputs == nullptr || output_count == nullptr)
    return fail(HYLE_HIP_INVALID_ARGUMENT, "null argument");
  for (uint32_t i = 0; i < plan->output_count; ++i) outputs[i] = plan->outputs[i];
  *output_count = plan->output_count;
  return HYLE_HIP_OK;
}

int hyle_hip_plan_alias_support(const hyle_hip_plan *plan, uint32_t output_index, uint32_t input_index) {
  if (plan == nullptr || output_index >= plan->output_count ||
      input_index >= plan->request.input_count)
    return 0;
  return (plan->alias_inputs[output_index] >> input_index) & 1u;
}

uint32_t hyle_hip_plan_dispatch_count(const hyle_hip_plan *plan) { return plan ? plan->dispatches : 0; }

const char *hyle_hip_plan_route_name(const hyle_hip_plan *plan) {
  if (plan == nullptr) return "";
  if (plan->route == Route::kReduce) {
    switch (plan->reduce.form) {
      case ReduceForm::kRows: return plan->reduce.tiles > 1 ? "reduce-row-tiles" : "reduce-rows";
      case ReduceForm::kColumns:
        return plan->reduce.segments > 1 ? "reduce-column-segments" : "reduce-columns";
      case ReduceForm::kGeneral: return "reduce-strided";
    }
  }
  if (plan->route == Route::kTopK && plan->topk.select) return "topk-select-tiles";
  return route_name(plan->route);
}

uint32_t hyle_hip_variant_count(void) {
  VariantList &list = variant_list();
  std::lock_guard<std::mutex> lock(list.mutex);
  return (uint32_t)list.labels.size();
}

const char *hyle_hip_variant_label(uint32_t index) {
  VariantList &list = variant_list();
  std::lock_guard<std::mutex> lock(list.mutex);
  return index < list.labels.size() ? list.labels[index]->c_str() : "";
}

const char *hyle_hip_last_launch_variant(void) {
  size_t used = 0;
  g_noted_text[0] = 0;
  for (int i = 0; i < g_noted_count; ++i) {
    const int wrote = snprintf(g_noted_text + used, sizeof g_noted_text - used, "%s%s", i ? " + " : "", g_noted[i]);
    if (wrote < 0 || (size_t)wrote >= sizeof g_noted_text - used) break;
    used += (size_t)wrote;
  }
  return g_noted_text;
}

hyle_hip_status hyle_hip_plan_launch(const hyle_hip_plan *plan, const void *const *inputs,
                                     uint32_t input_count, void *const *outputs, uint32_t output_count,
                                     void *workspace, size_t workspace_size, void *stream_handle) {
  g_noted_count = 0;
  if (plan == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "plan is null");
  if (input_count != plan->request.input_count || output_count != plan->output_count)
    return fail(HYLE_HIP_INVALID_ARGUMENT, "launch binding counts differ from the plan");
  if (plan->route == Route::kNoOp) return HYLE_HIP_OK;  // zero elements: storage is never touched
  if (plan->context == nullptr)
    return fail(HYLE_HIP_FAILED_PRECONDITION, "plan was built without a device context");
  if ((inputs == nullptr && input_count != 0) || outputs == nullptr)
    return fail(HYLE_HIP_INVALID_ARGUMENT, "binding arrays are null");
  bool vector = true;
  for (uint32_t i = 0; i < input_count; ++i) {
    if (plan->input_elements[i] == 0) continue;
    if (inputs[i] == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "input %u is null", i);
    if (!aligned(inputs[i], plan->input_alignment[i]))
      return fail(HYLE_HIP_FAILED_PRECONDITION, "input %u does not satisfy tensor alignment", i);
    // a one-element operand is read with a scalar load and never limits vector access
    if (plan->input_elements[i] > 1) vector = vector && aligned(inputs[i], 16);
  }
  for (uint32_t o = 0; o < output_count; ++o) {
    if (plan->output_elements[o] == 0) continue;
    if (outputs[o] == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "output %u is null", o);
    if (!aligned(outputs[o], plan->output_alignment[o]))
      return fail(HYLE_HIP_FAILED_PRECONDITION, "output %u does not satisfy tensor alignment", o);
    if (o == 0) vector = vector && aligned(outputs[o], 16);
    for (uint32_t i = 0; i < input_count; ++i)
      if (outputs[o] == inputs[i] && plan->input_elements[i] != 0 &&
          ((plan->alias_inputs[o] >> i) & 1u) == 0)
        return fail(HYLE_HIP_INVALID_ARGUMENT, "input %u cannot alias output %u on this route", i, o);
  }
  if (plan->workspace_size != 0) {
    if (workspace == nullptr || workspace_size < plan->workspace_size)
      return fail(HYLE_HIP_INVALID_ARGUMENT, "workspace is smaller than the plan requires");
    if (!aligned(workspace, plan->workspace_alignment))
      return fail(HYLE_HIP_FAILED_PRECONDITION, "workspace does not satisfy its alignment");
  }
  if (plan->no_overlap_output_bytes != 0) {
    const uintptr_t in_first = reinterpret_cast<uintptr_t>(inputs[0]), out_first = reinterpret_cast<uintptr_t>(outputs[0]);
    if (in_first < out_first + plan->no_overlap_output_bytes && out_first < in_first + plan->no_overlap_input_bytes)
      return fail(HYLE_HIP_INVALID_ARGUMENT, "input and output storage overlap; Cast and Copy take no alias");
  }
  hipStream_t stream = static_cast<hipStream_t>(stream_handle);
  hipError_t err = hipSuccess;
  switch (plan->route) {
    case Route::kNoOp: break;
    case Route::kEwFlat:
      err = launch_ew_flat(plan->elem, plan->flat, inputs[0], input_count > 1 ? inputs[1] : nullptr,
                           input_count > 2 ? inputs[2] : nullptr, outputs[0], vector, stream);
      break;
    case Route::kEwGeneral:
      err = launch_ew_general(plan->elem, plan->general, inputs[0],
                              input_count > 1 ? inputs[1] : nullptr,
                              input_count > 2 ? inputs[2] : nullptr, outputs[0], stream);
      break;
    case Route::kSwigluPacked:
      err = launch_swiglu_packed(plan->elem, plan->packed, inputs[0], outputs[0], vector, stream);
      break;
    case Route::kRmsNorm:
      err = launch_norm(plan->elem, plan->norm, inputs[0], input_count > 1 ? inputs[1] : nullptr,
                        input_count > 2 ? inputs[2] : nullptr, outputs[0], vector, stream);
      break;
    case Route::kSoftmax: {
      const void *mask = input_count > 1 ? inputs[1] : nullptr;
      const int kvec = elem_vec(plan->elem);
      const bool rows = plan->softmax_rows_ok && plan->softmax_mask_vector_ok &&
                        aligned(inputs[0], 16) && aligned(outputs[0], 16) &&
                        (mask == nullptr || aligned(mask, 16)) &&
                        plan->softmax.shape.width % kvec == 0 &&
                        plan->softmax.shape.width / kvec <= 8u * 1024u;  // the widest row shape: 1024 lanes x 8 vectors
      if (rows)
        err = launch_softmax(plan->elem, plan->softmax, inputs[0], mask, outputs[0], true,
                             plan->context->compute_units, stream);
      else
        err = launch_softmax_general(plan->elem, plan->softmax_general, inputs[0], mask, outputs[0],
                                     stream);
      break;
    }
    case Route::kReduce:
      err = launch_reduce(plan->elem, plan->reduce, inputs[0], outputs[0], workspace,
                          inputs[0] == nullptr || aligned(inputs[0], 16), stream);
      break;
    case Route::kArgmax:
      err = launch_argmax(plan->elem, plan->argmax, inputs[0], outputs[0],
                          static_cast<int32_t *>(outputs[1]), workspace, aligned(inputs[0], 16), stream);
      break;
    case Route::kTopK:
      err = launch_topk(plan->elem, plan->topk, inputs[0], outputs[0], static_cast<int32_t *>(outputs[1]),
                        workspace, aligned(inputs[0], 16), stream);
      break;
    case Route::kQ8Dequant:
      err = launch_q8_0_dequant(plan->q8, inputs[0], outputs[0], static_cast<float *>(outputs[1]),
                                aligned(inputs[0], 16) && aligned(outputs[0], 16), stream);
      break;
    case Route::kKQuantDequant:
      err = launch_k_quant_dequant(plan->kquant, inputs[0], outputs[0], static_cast<float *>(outputs[1]), stream);
      break;
    case Route::kGgufMatVec:
      if (plan->matvec.codec == HYLE_HIP_ACTIVATIONS_GGML_Q8)
        err = launch_gguf_matvec_q8(plan->elem, plan->matvec, inputs[0], inputs[1], outputs[0],
                                    plan->context->compute_units, stream);
      else
        err = launch_gguf_matvec(plan->elem, plan->matvec, inputs[0], inputs[1], outputs[0], stream);
      break;
    case Route::kCast:
      err = launch_cast(plan->cast, inputs[0], outputs[0], vector, stream);
      break;
    case Route::kFill:
      err = launch_fill(plan->fill, outputs[0], stream);
      break;
    case Route::kSelect:
      err = launch_select(plan->select, inputs[0], inputs[1], inputs[2], outputs[0], vector, stream);
      break;
    case Route::kConcat: {
      const uintptr_t out_first = reinterpret_cast<uintptr_t>(outputs[0]);
      const uint64_t out_bytes = plan->output_elements[0] * plan->concat.size;
      for (uint32_t i = 0; i < input_count; ++i) {
        if (plan->input_elements[i] == 0) continue;
        const uintptr_t in_first = reinterpret_cast<uintptr_t>(inputs[i]);
        if (in_first < out_first + out_bytes && out_first < in_first + plan->concat_input_bytes[i])
          return fail(HYLE_HIP_INVALID_ARGUMENT, "input %u and output storage overlap; Concat takes no alias", i);
      }
      err = launch_concat(plan->concat, inputs, outputs[0], stream);
      break;
    }
    case Route::kGather: {
      // src/compute_provider_native/indexing.cc:189-195
      if (plan->gather.extent == 0) return fail(HYLE_HIP_OUT_OF_RANGE, "Gather cannot index an empty axis");
      const uintptr_t out_first = reinterpret_cast<uintptr_t>(outputs[0]);
      const uint64_t out_bytes = plan->output_elements[0] * plan->gather.size;
      for (uint32_t i = 0; i < 2; ++i) {
        const uintptr_t in_first = reinterpret_cast<uintptr_t>(inputs[i]);
        if (in_first < out_first + out_bytes && out_first < in_first + plan->concat_input_bytes[i])
          return fail(HYLE_HIP_INVALID_ARGUMENT, "input %u and output storage overlap; Gather takes no alias", i);
      }
      err = launch_gather(plan->gather, inputs[0], inputs[1], outputs[0], workspace, stream);
      break;
    }
    case Route::kRope:
      err = launch_rope(plan->elem, plan->rope, inputs[0], inputs[1], inputs[2], outputs[0],
                        aligned(inputs[0], 16) && aligned(outputs[0], 16), stream);
      break;
    case Route::kRandomBits:
      err = launch_random_bits(plan->random_bits, inputs[0], outputs[0], stream);
      break;
    case Route::kCategorical:
      err = launch_categorical(plan->elem, plan->categorical, inputs[0], inputs[1], outputs[0],
                               output_count > 1 ? outputs[1] : nullptr, workspace, aligned(inputs[0], 16), stream);
      break;
  }
  if (err != hipSuccess) return hip_fail(err, "kernel launch");
  return HYLE_HIP_OK;
}

int hyle_hip_plan_device_status_offset(const hyle_hip_plan *plan, size_t *offset) {
  if (plan == nullptr) return 0;
  if (plan->route == Route::kGather && plan->gather.checked) {
    if (offset != nullptr) *offset = (size_t)kGatherStatusWord * 4;
    return 1;
  }
  if (plan->route == Route::kCategorical) {
    if (offset != nullptr) *offset = plan->categorical.status_offset;
    return 1;
  }
  return 0;
}

hyle_hip_status hyle_hip_plan_device_status(const hyle_hip_plan *plan, const void *workspace, void *stream_handle) {
  if (plan == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "plan is null");
  size_t offset = 0;
  if (!hyle_hip_plan_device_status_offset(plan, &offset)) return HYLE_HIP_OK;
  if (workspace == nullptr) workspace = plan->context != nullptr ? plan->context->static_scratch : nullptr;
  if (workspace == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "workspace is null");
  hipStream_t stream = static_cast<hipStream_t>(stream_handle);
  uint32_t word = 0;
  hipError_t err = hipMemcpyAsync(&word, static_cast<const unsigned char *>(workspace) + offset, sizeof(word),
                                  hipMemcpyDeviceToHost, stream);
  if (err == hipSuccess) err = hipStreamSynchronize(stream);
  if (err != hipSuccess) return hip_fail(err, "reading the device status word");
  if (word == kStatusIndexOutOfRange) return fail(HYLE_HIP_OUT_OF_RANGE, "Gather index is outside the selected axis");
  if (word == kStatusInvalidNumericInput)
    return fail(HYLE_HIP_INVALID_ARGUMENT, "Categorical requires valid nonzero row mass");
  if (word != 0) return fail(HYLE_HIP_INTERNAL, "device status word holds %u", word);
  return HYLE_HIP_OK;
}

size_t hyle_hip_static_scratch_bytes(void) { return kStaticScratchBytes; }

hyle_hip_status hyle_hip_plan_launch_static(const hyle_hip_plan *plan, const void *const *inputs,
                                            uint32_t input_count, void *const *outputs, uint32_t output_count,
                                            void *stream_handle) {
  g_noted_count = 0;
  if (plan == nullptr) return fail(HYLE_HIP_INVALID_ARGUMENT, "plan is null");
  if (plan->workspace_size > kStaticScratchBytes)
    return fail(HYLE_HIP_RESOURCE_EXHAUSTED,
                "the plan needs %zu bytes of workspace; the device scratch of hyle_hip_plan_launch_static holds %zu: "
                "use hyle_hip_plan_launch with a caller-owned workspace",
                plan->workspace_size, kStaticScratchBytes);
  void *workspace = nullptr;
  if (plan->workspace_size != 0) {
    if (plan->context == nullptr || plan->context->static_scratch == nullptr)
      return fail(HYLE_HIP_FAILED_PRECONDITION, "plan was built without a device context");
    workspace = plan->context->static_scratch;
  }
  // Every route writes the part of the workspace it later reads, so nothing has to start at
  // zero; the last call's contents are simply overwritten.
  return hyle_hip_plan_launch(plan, inputs, input_count, outputs, output_count, workspace,
                              plan->workspace_size, stream_handle);
}

}  // extern "C"

// Hooks for the other translation units of the library (file_stream.hip): the device a context
// is bound to, and the per-thread error text behind hyle_hip_last_error.
namespace hyle_hip {
int context_device(const hyle_hip_context *context) { return context ? context->device : -1; }
int record_error(int status, const char *text) {
  return fail(static_cast<hyle_hip_status>(status), "%s", text);
}
}  // namespace hyle_hip
