/*
 * hyle_hip.h -- C ABI of the MI355X (gfx950) compute provider for HYLE's tensor
 * hot path: broadcast Binary, Unary SiLU, GatedActivation (SwiGLU), RMSNorm,
 * row Softmax / LogSoftmax, Reduce over any set of axes, TopK and Q8_0 block dequant.
 *
 * The surface is what a `hyle::compute` provider for this path binds: one cold
 * "plan" per (Operation, input descriptors) pair -- the reference's
 * propose + prepare -- and one allocation-free, non-blocking launch per
 * submit on a caller-owned HIP stream.  Plain pointers and sizes only.
 *
 * Enumerator values are the reference's own so that an adapter can cast:
 *   hyle_hip_status     <- hyle::StatusCode          (include/hyle/error/status.h:18-38)
 *   hyle_hip_dtype      <- hyle::compute::DataType   (include/hyle/compute/tensor_desc.h:17-34)
 *   hyle_hip_op_kind    <- hyle::compute::OperationKind (include/hyle/compute/operation.h:22-48)
 *   sub-kinds           <- UnaryKind / BinaryKind / ReductionKind /
 *                          GatedActivationKind / GatedInputKind / SoftmaxKind /
 *                          MaskKind (include/hyle/compute/operation.h:57-126)
 */
#ifndef HYLE_HIP_H_
#define HYLE_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#define HYLE_HIP_API __attribute__((visibility("default")))
#else
#define HYLE_HIP_API
#endif

#define HYLE_HIP_MAX_RANK 8      /* hyle::compute::kMaxTensorRank */
#define HYLE_HIP_MAX_INPUTS 4
#define HYLE_HIP_MAX_OUTPUTS 2
#define HYLE_HIP_ABI_VERSION 1u
/* Device scratch behind hyle_hip_plan_launch_static, per device. */
#define HYLE_HIP_STATIC_SCRATCH_BYTES (4u * 1024u * 1024u)

/* hyle::StatusCode.  UNIMPLEMENTED from plan_create is a clean decline (the
 * caller tries its next provider, src/compute/operation.cc:1259-1266); every
 * other non-OK code is an error. */
typedef enum hyle_hip_status {
  HYLE_HIP_OK = 0,
  HYLE_HIP_CANCELLED = 1, /* a file-pipeline request that was asked to stop (hyle_hip_stream.h) */
  HYLE_HIP_INVALID_ARGUMENT = 3,
  HYLE_HIP_RESOURCE_EXHAUSTED = 8,
  HYLE_HIP_FAILED_PRECONDITION = 9,
  HYLE_HIP_OUT_OF_RANGE = 11,
  HYLE_HIP_UNIMPLEMENTED = 12,
  HYLE_HIP_INTERNAL = 13,
  HYLE_HIP_UNAVAILABLE = 14
} hyle_hip_status;

/* hyle::compute::DataType (include/hyle/compute/tensor_desc.h:17-34).  Arithmetic serves F32 / F16 /
 * BF16 (TopK also I32, Cast also Bool and I32 sources); every type is storage for the operations
 * that only move bits (Copy, Fill, Select, Concat, Gather), and I32 / I64 index Gather. */
typedef enum hyle_hip_dtype {
  HYLE_HIP_DTYPE_UNKNOWN = 0,
  HYLE_HIP_DTYPE_BOOL = 1,
  HYLE_HIP_DTYPE_F8_E4M3FN = 2,
  HYLE_HIP_DTYPE_F8_E5M2 = 3,
  HYLE_HIP_DTYPE_F16 = 4,
  HYLE_HIP_DTYPE_BF16 = 5,
  HYLE_HIP_DTYPE_F32 = 6,
  HYLE_HIP_DTYPE_F64 = 7,
  HYLE_HIP_DTYPE_I8 = 8,
  HYLE_HIP_DTYPE_U8 = 9,
  HYLE_HIP_DTYPE_I16 = 10,
  HYLE_HIP_DTYPE_U16 = 11,
  HYLE_HIP_DTYPE_I32 = 12,
  HYLE_HIP_DTYPE_U32 = 13,
  HYLE_HIP_DTYPE_I64 = 14,
  HYLE_HIP_DTYPE_U64 = 15
} hyle_hip_dtype;

/* hyle::compute::RopeLayout (include/hyle/compute/operation.h:112-115): pairs are (2i, 2i + 1) or
 * (i, i + rotary / 2). */
typedef enum hyle_hip_rope_layout {
  HYLE_HIP_ROPE_INTERLEAVED = 0,
  HYLE_HIP_ROPE_HALF_SPLIT = 1
} hyle_hip_rope_layout;

/* hyle::compute::IndexBoundsPolicy (include/hyle/compute/operation.h:102-105) */
typedef enum hyle_hip_index_bounds {
  HYLE_HIP_BOUNDS_CHECKED = 0,
  HYLE_HIP_BOUNDS_UNCHECKED = 1
} hyle_hip_index_bounds;

typedef enum hyle_hip_op_kind {
  /* Copy: any plain input (dense or strided) materialised as a dense tensor of the same type.
   * Cast: the same with a change of storage type, `kind` = destination hyle_hip_dtype
   * (f32/f16/bf16 among each other, int32 -> f32, Bool <-> float; equal types copy).
   * Neither takes an alias: input and output bytes must not overlap. */
  HYLE_HIP_OP_COPY = 2,
  /* Fill (include/hyle/compute/operation.h: struct Fill): no inputs (input_count = 0).  The
   * output shape is the rank and dims of inputs[0] (its other fields are ignored), `kind` the
   * output hyle_hip_dtype, which is also the scalar's type, and `count` ScalarValue::bits():
   * the element's bit pattern in the low bytes. */
  HYLE_HIP_OP_FILL = 3,
  HYLE_HIP_OP_CAST = 4,
  HYLE_HIP_OP_UNARY = 5,
  HYLE_HIP_OP_BINARY = 6,
  /* Select: inputs (condition Bool, first, second), the three broadcast together; the output
   * holds `first` where the condition byte is non-zero and `second` elsewhere, bit for bit. */
  HYLE_HIP_OP_SELECT = 7,
  HYLE_HIP_OP_REDUCE = 8,
  HYLE_HIP_OP_RMS_NORM = 9,
  /* in0 [.., n], optional scale [n], optional bias [n] (bias only with a scale) */
  HYLE_HIP_OP_LAYER_NORM = 10,
  HYLE_HIP_OP_GATED_ACTIVATION = 12,
  /* Gather (include/hyle/compute/operation.h:367-370): in0 a plain source of any storage type,
   * in1 plain I32 / I64 indices of any rank; out0 is the source with `axis` replaced by the shape
   * of the indices, bits kept.  `kind2` = hyle_hip_index_bounds.  Checked bounds take two
   * dispatches and a small workspace: an index below 0 or at / past the axis extent leaves every
   * byte of the output as it was and shows as OUT_OF_RANGE in hyle_hip_plan_device_status once
   * the launch has completed.  Unchecked bounds take one dispatch and trust the caller.  No alias:
   * the output overlaps neither input. */
  HYLE_HIP_OP_GATHER = 13,
  /* Concat: 1..4 inputs of one type and rank joined along `axis` (negative counts from the end).
   * A caller with more inputs issues one plan per group of four into the same output: `kind` is
   * then the output's whole extent on the axis (0: the sum of this plan's inputs) and `count` the
   * place on the axis where this group starts; the plan writes only its own inputs' part. */
  HYLE_HIP_OP_CONCAT = 15,
  /* RoPE (include/hyle/compute/operation.h:388-392): in0 dense F32 / F16 / BF16 data of rank >= 2,
   * in1 dense I32 / I64 positions ([S] or the data's leading dimensions through the sequence
   * axis), in2 dense F32 frequencies ([rotary / 2] or [S, rotary / 2]); out0 like in0.  `count` =
   * rotary_dimensions (positive, even, at most the last extent), `axis` = sequence_axis (not the
   * last), `kind2` = hyle_hip_rope_layout.  Arithmetic in f32 with phase = frequency * f32(position);
   * elements past rotary_dimensions pass through.  out0 may alias in0. */
  HYLE_HIP_OP_ROPE = 16,
  HYLE_HIP_OP_SOFTMAX = 18,
  HYLE_HIP_OP_TOP_K = 19,
  /* Fused forms with no single counterpart in the reference schema; a HYLE
   * adapter reaches them through OperationKind::kCustom (24). */
  /* out = (in0 kind in1) kind2 in2, the intermediate rounded to the storage
   * type: bit-identical to two chained Binary operations. */
  HYLE_HIP_OP_BINARY_CHAIN = 0x100,
  /* in0: Q8_0 blocked weight, logical [K, N], physical rows of K/32 blocks;
   * out0: bf16 [N, K] dense; out1: f32 [N] row sum of squares of the exact
   * f32 products. */
  HYLE_HIP_OP_Q8_0_DEQUANT_SUMSQ = 0x101,
  /* The same operation under its general name: the weight may also be GGUF Q4_K (256-element,
   * 144-byte blocks) or Q6_K (256-element, 210-byte blocks); the block geometry of in0 selects
   * the decoder (src/compute_ops/low_precision.cc:22-29). */
  HYLE_HIP_OP_GGUF_DEQUANT_SUMSQ = 0x101,
  /* MatMul(in1, in0) for token-by-token decoding: in0 a GGUF weight (Q8_0, Q4_K, Q6_K), logical
   * [K, N]; in1 dense f32 / f16 / bf16 activations [K] or [M, K] with M <= 8; out0 [N] or [M, N]
   * of in1's type.  kind2 selects the arithmetic (HYLE_HIP_ACTIVATIONS_*): EXACT decodes the
   * weights exactly and multiplies in f32; GGML_Q8 is what the reference's ggml CPU route
   * computes: the activations are first quantised to ggml's 8-bit blocks (Q8_0 blocks for a Q8_0
   * weight, Q8_K blocks for Q4_K / Q6_K) and the block dot products are integers
   * (tests/compute_models/qwen27_original_nextn_reference.h:94-167,193-257 holds that
   * arithmetic and the bound the reference accepts of it). */
  HYLE_HIP_OP_GGUF_MATVEC = 0x102,
  /* sampling_ops::RandomBits (include/hyle/compute/sampling_ops.h:12-35): in0 dense U32 [R, 4]
   * identities (key low / high, draw low / high), `count` = word_count; out0 dense U32
   * [R, word_count] of Philox4x32-10 words, word j = lane j % 4 of the block with counter
   * {j / 4, draw}.  Bit for bit the words of every backend of the reference. */
  HYLE_HIP_OP_RANDOM_BITS = 0x103,
  /* sampling_ops::Categorical (include/hyle/compute/sampling_ops.h:37-66): in0 dense F32 / F16 /
   * BF16 [R, V] log-weights, in1 dense U32 [R, 4] identities; out0 I32 [R] indices and, with
   * `kind2` = 1, out1 F32 [R] normalised log probabilities of the selected elements.  -Inf is
   * zero mass.  Two dispatches and a workspace; a row with NaN, +Inf or no finite element writes
   * nothing and shows as INVALID_ARGUMENT in hyle_hip_plan_device_status.  The draw is the CPU
   * provider's inverse CDF on the 52-bit uniform of the row's first Philox block; like the
   * reference's own backends it promises the distribution, not equal indices across backends. */
  HYLE_HIP_OP_CATEGORICAL = 0x104
} hyle_hip_op_kind;

/* UnaryKind (include/hyle/compute/operation.h:57-73) */
enum {
  HYLE_HIP_UNARY_ABS = 0,
  HYLE_HIP_UNARY_NEG = 1,
  HYLE_HIP_UNARY_EXP = 2,
  HYLE_HIP_UNARY_LOG = 3,
  HYLE_HIP_UNARY_SQRT = 4,
  HYLE_HIP_UNARY_RSQRT = 5,
  HYLE_HIP_UNARY_TANH = 6,
  HYLE_HIP_UNARY_SIGMOID = 7,
  HYLE_HIP_UNARY_RELU = 8,
  HYLE_HIP_UNARY_GELU = 9,
  HYLE_HIP_UNARY_GELU_TANH = 10,
  HYLE_HIP_UNARY_SILU = 11,
  HYLE_HIP_UNARY_SOFTPLUS = 12
};
/* BinaryKind (include/hyle/compute/operation.h:75-82) */
enum {
  HYLE_HIP_BINARY_ADD = 0,
  HYLE_HIP_BINARY_SUBTRACT = 1,
  HYLE_HIP_BINARY_MULTIPLY = 2,
  HYLE_HIP_BINARY_DIVIDE = 3,
  HYLE_HIP_BINARY_MINIMUM = 4,
  HYLE_HIP_BINARY_MAXIMUM = 5
};
/* ReductionKind (include/hyle/compute/operation.h:84-89) */
enum {
  HYLE_HIP_REDUCE_SUM = 0,
  HYLE_HIP_REDUCE_MEAN = 1,
  HYLE_HIP_REDUCE_MINIMUM = 2,
  HYLE_HIP_REDUCE_MAXIMUM = 3
};
/* GatedActivationKind / GatedInputKind (include/hyle/compute/operation.h:91-100) */
enum { HYLE_HIP_GATED_SILU = 0, HYLE_HIP_GATED_GELU = 1, HYLE_HIP_GATED_GELU_TANH = 2 };
enum { HYLE_HIP_GATED_PACKED_HALVES = 0, HYLE_HIP_GATED_SEPARATE = 1 };
/* SoftmaxKind / MaskKind (include/hyle/compute/operation.h:117-126) */
enum { HYLE_HIP_SOFTMAX = 0, HYLE_HIP_LOG_SOFTMAX = 1 };
enum { HYLE_HIP_MASK_NONE = 0, HYLE_HIP_MASK_ADDITIVE = 1, HYLE_HIP_MASK_BOOLEAN = 2 };

/* GGUF_MATVEC kind2 */
enum { HYLE_HIP_ACTIVATIONS_EXACT = 0, HYLE_HIP_ACTIVATIONS_GGML_Q8 = 1 };

/* StorageFormatKind (include/hyle/compute/tensor_desc.h:77-81) */
enum { HYLE_HIP_STORAGE_PLAIN = 0, HYLE_HIP_STORAGE_BLOCKED = 1 };

/* hyle::compute::TensorDesc as plain data
 * (include/hyle/compute/tensor_desc.h:141-225): logical dims, BYTE strides, a
 * zero stride on an axis of extent > 1 is a broadcast; blocked storage names
 * its block axis and block geometry. */
typedef struct hyle_hip_tensor_desc {
  uint8_t dtype;        /* hyle_hip_dtype */
  uint8_t rank;         /* 0..8 */
  uint8_t storage;      /* HYLE_HIP_STORAGE_* */
  uint8_t block_axis;   /* valid when storage == BLOCKED */
  uint32_t elements_per_block;
  uint32_t bytes_per_block;
  uint32_t reserved;
  int64_t dims[HYLE_HIP_MAX_RANK];
  int64_t byte_strides[HYLE_HIP_MAX_RANK];
} hyle_hip_tensor_desc;

/* One hyle::compute::Operation plus its exact input descriptors
 * (ProviderOperationRequest, src/compute/provider_internal.h:45-53). */
typedef struct hyle_hip_op_desc {
  uint32_t abi_version;      /* HYLE_HIP_ABI_VERSION */
  uint32_t op;               /* hyle_hip_op_kind */
  uint32_t kind;             /* Unary/Binary/Reduction/GatedActivation kind; Cast, Fill: output hyle_hip_dtype */
  uint32_t kind2;            /* BINARY_CHAIN: second BinaryKind; GATED: GatedInputKind;
                                SOFTMAX: SoftmaxKind; GGUF_MATVEC: HYLE_HIP_ACTIVATIONS_*;
                                GATHER: hyle_hip_index_bounds; CATEGORICAL: 1 = also log probabilities;
                                ROPE: hyle_hip_rope_layout */
  int32_t axis;              /* Softmax / TopK / Concat / Gather axis, RoPE sequence axis (negative counts from the end) */
  uint32_t mask;             /* Softmax MaskKind */
  uint32_t accumulation;     /* hyle_hip_dtype; UNKNOWN or F32 */
  uint32_t keep_dimensions;  /* Reduce */
  float epsilon;             /* RmsNorm, LayerNorm */
  float scale;               /* Softmax */
  uint64_t count;            /* TopK count; Fill: the scalar's bits; Concat: the group's start on the axis;
                                RandomBits: word_count; RoPE: rotary_dimensions */
  uint32_t largest;          /* TopK: 1 = largest first, 0 = smallest first */
  uint32_t input_count;
  hyle_hip_tensor_desc inputs[HYLE_HIP_MAX_INPUTS];
  /* Reduce::axes (include/hyle/compute/operation.h:232-247, 307-312): axes_count = 0 is
   * Axes::all(); otherwise the first axes_count entries of `axes`, each possibly negative
   * (counted from the end); a duplicate is INVALID_ARGUMENT as in the schema
   * (src/compute_ops/operation.cc:1358-1377). */
  uint32_t axes_count;
  int32_t axes[HYLE_HIP_MAX_RANK];
} hyle_hip_op_desc;

typedef struct hyle_hip_context hyle_hip_context;
typedef struct hyle_hip_plan hyle_hip_plan;

/* ProviderVTable::create_context / destroy_context
 * (src/compute/provider_internal.h:124-129).  Binds one HIP device; fails with
 * UNAVAILABLE when no gfx950 device is present. */
HYLE_HIP_API hyle_hip_status hyle_hip_context_create(int device, hyle_hip_context **context);
HYLE_HIP_API void hyle_hip_context_destroy(hyle_hip_context *context);
/* Compute units of the bound device. */
HYLE_HIP_API int hyle_hip_context_compute_units(const hyle_hip_context *context);

/* Provider-neutral output inference, hyle::compute::infer_output_descriptions
 * (src/compute_ops/operation.cc:1214-1704) for the operations above.  Needs no
 * device.  Writes up to HYLE_HIP_MAX_OUTPUTS descriptors. */
HYLE_HIP_API hyle_hip_status hyle_hip_infer_outputs(const hyle_hip_op_desc *request,
                                                    hyle_hip_tensor_desc *outputs,
                                                    uint32_t *output_count);

/* ProviderVTable::propose + prepare (src/compute/provider_internal.h:130-142):
 * validates the request against the schema, then admits it into a kernel route.
 * `outputs` may be NULL (inferred dense outputs) or the caller's exact output
 * descriptors, which must equal the inferred ones. */
HYLE_HIP_API hyle_hip_status hyle_hip_plan_create(hyle_hip_context *context,
                                                  const hyle_hip_op_desc *request,
                                                  const hyle_hip_tensor_desc *outputs,
                                                  uint32_t output_count, hyle_hip_plan **plan);
/* ProviderPreparedVTable::destroy_prepared
 * (include/hyle/compute/detail/prepared_callbacks.h:15-16). */
HYLE_HIP_API void hyle_hip_plan_destroy(hyle_hip_plan *plan);

/* ProviderPrepared::workspace (src/compute/provider_internal.h:85-88):
 * caller-owned device scratch the launch needs; size 0 for most routes. */
HYLE_HIP_API hyle_hip_status hyle_hip_plan_workspace(const hyle_hip_plan *plan, size_t *size,
                                                     size_t *alignment);
/* The inferred output descriptors of a plan. */
HYLE_HIP_API hyle_hip_status hyle_hip_plan_outputs(const hyle_hip_plan *plan,
                                                   hyle_hip_tensor_desc *outputs,
                                                   uint32_t *output_count);
/* ProviderPreparedVTable::alias_support
 * (include/hyle/compute/detail/prepared_callbacks.h:17-18): 1 when output
 * `output_index` may share exact storage with input `input_index`. */
HYLE_HIP_API int hyle_hip_plan_alias_support(const hyle_hip_plan *plan, uint32_t output_index,
                                             uint32_t input_index);
/* ProviderRouteCostFacts::dispatch_count
 * (include/hyle/compute/prepared_operation.h:51-67): kernels one launch enqueues. */
HYLE_HIP_API uint32_t hyle_hip_plan_dispatch_count(const hyle_hip_plan *plan);
/* Name of the kernel route the plan selected (diagnostics, profiling). */
HYLE_HIP_API const char *hyle_hip_plan_route_name(const hyle_hip_plan *plan);

/* Diagnostics for tests and profiling; no counterpart in the reference.  Inside a route the
 * launcher picks a kernel shape from the sizes, strides and alignments it sees at launch.  Every
 * shape compiled into the library has a label ("softmax_rows/512x2/additive/exact/steered");
 * hyle_hip_variant_count / hyle_hip_variant_label list them, and hyle_hip_last_launch_variant
 * returns the label(s) of the dispatches the calling thread's last hyle_hip_plan_launch or
 * hyle_hip_plan_launch_static enqueued, joined by " + " (empty when it enqueued nothing; consecutive
 * dispatches of one shape are one entry; at most four entries).  The text stays valid until the
 * thread's next call of the same function. */
HYLE_HIP_API uint32_t hyle_hip_variant_count(void);
HYLE_HIP_API const char *hyle_hip_variant_label(uint32_t index);
HYLE_HIP_API const char *hyle_hip_last_launch_variant(void);

/* ProviderPreparedVTable::shared_submit
 * (include/hyle/compute/detail/prepared_callbacks.h:26-30): enqueue on `stream`
 * (a hipStream_t; NULL is the default stream) and return without waiting.
 * Pointers are device addresses of the tensors' first logical element.  No
 * allocation, no synchronisation.  A non-OK return means nothing was enqueued
 * (EnqueueResult::rejected).  Zero-element tensors succeed without touching
 * storage. */
HYLE_HIP_API hyle_hip_status hyle_hip_plan_launch(const hyle_hip_plan *plan,
                                                  const void *const *inputs, uint32_t input_count,
                                                  void *const *outputs, uint32_t output_count,
                                                  void *workspace, size_t workspace_size,
                                                  void *stream);

/* The device-side verdict of a launch whose kernels can refuse their input: checked Gather, whose
 * reference counterpart fails the Completion with OutOfRange when an index lies outside the axis
 * (src/compute_provider_cuda/collectives.cu:123-145; tests/compute_provider_cuda/
 * gather_collectives_test.cc:176-212), and Categorical, which fails it with InvalidArgument for a
 * row without valid mass (src/compute_provider_cuda/sampling_kernel.cu:47-79).  Waits for `stream`, reads the plan's status word from
 * `workspace` (the one the launch was given; NULL after hyle_hip_plan_launch_static) and returns
 * OK, OUT_OF_RANGE or INVALID_ARGUMENT.  Plans without such a word return OK at once, without waiting.  An adapter
 * calls this from Completion::wait; hyle_hip_plan_device_status_offset gives the word's place in
 * the workspace (a uint32, non-zero = refused) for one that prefers its own asynchronous copy,
 * and returns 0 when the plan has no such word. */
HYLE_HIP_API hyle_hip_status hyle_hip_plan_device_status(const hyle_hip_plan *plan, const void *workspace,
                                                         void *stream);
HYLE_HIP_API int hyle_hip_plan_device_status_offset(const hyle_hip_plan *plan, size_t *offset);

/* hyle_hip_plan_launch for callers that cannot allocate device memory and have no workspace to
 * pass: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It
 * has no counterpart in the reference, whose callers always own the workspace
 * (ProviderPrepared::workspace).  The workspace of the two-dispatch routes (TopK, tiled Reduce)
 * is a file-scope device array of HYLE_HIP_STATIC_SCRATCH_BYTES that every device holds from
 * the first context on it until the process ends; its address is looked up once per device in
 * hyle_hip_context_create.  Nothing is allocated or freed here.  A plan whose workspace exceeds
 * the array is refused with RESOURCE_EXHAUSTED.  All calls on one device share the one array:
 * calls that may overlap on a device (different streams, different threads) race, so serialise
 * them on one stream or use hyle_hip_plan_launch with separate workspaces.  Results are those of
 * hyle_hip_plan_launch bit for bit.  The device verdict of a checked Gather or a Categorical
 * launched this way lives in that shared array too: read it with
 * hyle_hip_plan_device_status(plan, NULL, stream) before the next static launch on the device,
 * which may overwrite it (the next launch of any plan with a workspace, even on the same stream). */
HYLE_HIP_API hyle_hip_status hyle_hip_plan_launch_static(const hyle_hip_plan *plan,
                                                         const void *const *inputs, uint32_t input_count,
                                                         void *const *outputs, uint32_t output_count,
                                                         void *stream);
/* Size of that array: the largest hyle_hip_plan_workspace a plan may need to be served. */
HYLE_HIP_API size_t hyle_hip_static_scratch_bytes(void);

/* Text of the last non-OK status returned on the calling thread. */
HYLE_HIP_API const char *hyle_hip_last_error(void);
HYLE_HIP_API const char *hyle_hip_status_name(hyle_hip_status status);
HYLE_HIP_API uint32_t hyle_hip_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* HYLE_HIP_H_ */
