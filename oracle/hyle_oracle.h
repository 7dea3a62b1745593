/*
 * hyle_oracle.h -- CPU restatement of the reference's scalar semantics for the
 * tensor hot path (broadcast add/mul, SiLU, SwiGLU, RMSNorm, row softmax, row
 * max/sum, argmax, Q8_0 block decode).
 *
 * THIS IS TEST INFRASTRUCTURE.  It is the checker the HIP kernels are compared
 * against and the "port" CPU baseline that bench.py times beside the GPU; it
 * is never linked into, loaded by, or called from the shipped library.
 *
 * Every function cites the reference file:line it follows (paths relative to
 * the reference tree).  Storage types f16/bf16 are carried as uint16_t bit
 * patterns.  Built with -ffp-contract=off: a fused multiply-add happens only
 * where the reference itself writes std::fma.
 *
 * Parity status (what pins each function is listed in oracle/README.md):
 *   - codecs, silu, swiglu, rms_norm (scalar floor), softmax: pinned bit-exact
 *     against the reference's own scalar floor compiled from its sources
 *     (oracle/_ref), plus the reference tests' known-answer vectors.
 *   - binary add/mul, broadcast offsets, reduce, index_of_max, topk1: pinned by
 *     IEEE closed forms, brute force and the reference tests' known answers.
 *   - q8_0 decode: restated from the block format, pinned by an exactness
 *     argument with exhaustive scale x quant enumeration against an independent
 *     integer/double evaluation, and by the element values the reference's own
 *     tests expect (see k_quant_dequant below).
 *   - rms_norm_bf16_native tile order: "parity unpinned" at the bit level (the
 *     reference sums each 128-wide tile with a Highway vector dot whose lane
 *     order is target-dependent); pinned only to tolerance.
 *   - cast, layer_norm, unary / gated kinds, reduce over any axes, topk:
 *     pinned by the reference's scalar floor (where it holds the function),
 *     its tests' known answers and numpy / float64 closed forms.
 *   - log_softmax: the floor's form (log_softmax_floor) is pinned bit-exact
 *     against oracle/_ref and golden vectors; the log1p form the GPU kernel
 *     follows is held to it at the reference's own bound.
 *   - k_quant_dequant (GGUF Q4_K, Q6_K) and q8_0 decode: ggml's source is not
 *     in the reference tree, but two independent readings of the formats are
 *     (third_party/ggml_q4k_apple/ggml_q4k_apple.h:9-38; the element values of
 *     tests/compute_models/qwen27_original_nextn_reference.h:74-86,262-287):
 *     pinned bit for bit against both over random raw bytes, and against
 *     blocks packed field by field.
 *   - gguf_matvec_q8 (MatMul as the reference's ggml route computes it): the
 *     8-bit activation codecs, the centre and the bound are the ones the
 *     reference's tests hold for that route; pinned against array-wise
 *     restatements of those forms and a float64 product of independently
 *     decoded weights.  No output vector of ggml itself exists in the tree, so
 *     agreement is to the tests' bound, not bit for bit: PARITY UNPINNED at the
 *     bit level.  gguf_matvec (exact weights, double accumulation) is the
 *     mathematical product and is what the bound is centred on.
 *   - fill, select: the reference route test's expectation
 *     (tests/compute_route_vulkan/tensor_test.cc:255-283) and numpy's
 *     broadcasting `where` over raw words.
 *   - concat_part: numpy.concatenate over raw words in the shape of the
 *     reference route test (tests/compute_route_vulkan/concat_test.cc:9-88).
 *   - rope: the reference tests' known answers (tests/compute_provider_ggml/
 *     cpu_provider_test.cc:1571-1760, incl. the long-position phases), a
 *     float64 rotation, and what rotations obey (zero position or frequency is
 *     the identity, norms of pairs are kept, the tail passes through).  libm's
 *     cosf / sinf stand for ggml's: agreement is to tolerance, PARITY UNPINNED
 *     at the bit level.
 *   - philox_block, random_bits: the published Random123 known-answer vectors
 *     for philox4x32_10 and the independent array form in the reference's
 *     tests (tests/compute_models/sampling_fixture.h:70-91).
 *   - categorical: restated from the CPU recipe; checked against a float64
 *     inverse-CDF in numpy, the reference test's properties (one positive
 *     mass, row permutation, score within 2e-5 of the float64 normaliser,
 *     tests/compute_models/sampling_fixture.h:153-283) and its seven-sigma
 *     quality gate.  Selected indices need not match across the reference's
 *     own backends (include/hyle/compute/sampling_ops.h:50-55).
 *   - gather: numpy.take over raw words in the shape of the reference tests
 *     (tests/compute_provider_cuda/gather_collectives_test.cc,
 *     collectives_test_support.h:257-314) and their checked-failure cases.
 */
#ifndef HYLE_ORACLE_H_
#define HYLE_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HYLE_ORACLE_MAX_RANK 8

/* element types understood by the typed entry points */
enum {
  HYLE_ORACLE_F32 = 0,
  HYLE_ORACLE_F16 = 1,
  HYLE_ORACLE_BF16 = 2,
  /* Cast only */
  HYLE_ORACLE_BOOL = 3,
  HYLE_ORACLE_I32 = 4,
};

/* include/hyle/compute/operation.h:75-82 */
enum {
  HYLE_ORACLE_ADD = 0,
  HYLE_ORACLE_SUBTRACT = 1,
  HYLE_ORACLE_MULTIPLY = 2,
  HYLE_ORACLE_DIVIDE = 3,
  HYLE_ORACLE_MINIMUM = 4,
  HYLE_ORACLE_MAXIMUM = 5,
};

/* include/hyle/compute/operation.h:84-89 */
enum {
  HYLE_ORACLE_SUM = 0,
  HYLE_ORACLE_MEAN = 1,
  HYLE_ORACLE_MIN = 2,
  HYLE_ORACLE_MAX = 3,
};

/* include/hyle/compute/operation.h:122-126 */
enum {
  HYLE_ORACLE_MASK_NONE = 0,
  HYLE_ORACLE_MASK_ADDITIVE = 1,
  HYLE_ORACLE_MASK_BOOLEAN = 2,
};

/* ---- codecs: include/hyle/simd/dtype.h:55-121 --------------------------- */
float hyle_oracle_f16_to_f32(uint16_t bits);
uint16_t hyle_oracle_f32_to_f16(float value);
float hyle_oracle_bf16_to_f32(uint16_t bits);
uint16_t hyle_oracle_f32_to_bf16(float value);
void hyle_oracle_convert_to_f32(int type, const void *src, float *dst, size_t n);
void hyle_oracle_convert_from_f32(int type, const float *src, void *dst, size_t n);

/* ---- shape helpers ------------------------------------------------------ */
/* src/compute_ops/operation.cc:249-278.  Returns the result rank, or -1 when
 * the shapes cannot be broadcast / the rank exceeds 8. */
int hyle_oracle_broadcast_shape(const int64_t *left, int left_rank,
                                const int64_t *right, int right_rank,
                                int64_t *out);
/* src/compute_provider_native/native_plan.h:152-174 */
size_t hyle_oracle_broadcast_byte_offset(const int64_t *in_dims,
                                         const int64_t *in_strides, int in_rank,
                                         const int64_t *out_dims, int out_rank,
                                         size_t linear_index);
/* src/compute_provider_native/native_plan.h:135-147 */
size_t hyle_oracle_logical_byte_offset(const int64_t *dims,
                                       const int64_t *strides, int rank,
                                       size_t linear_index);

/* ---- elementwise -------------------------------------------------------- */
/* Scalar semantic of one Binary kind on f32 operands
 * (src/compute_provider_native/elementwise.cc:102-114; Multiply and Maximum
 * from tests/compute_provider_native/elementwise_test.cc:84-101). */
float hyle_oracle_binary_scalar(int kind, float left, float right);

/* Broadcasting Binary: dense output of out_rank dims, inputs described by
 * dims + byte strides (zero stride on a broadcast axis is honoured through
 * the "input dimension == 1" rule of the reference).  Storage type `type`;
 * narrow types decode -> f32 op -> one RN-even store
 * (src/compute_provider_native/elementwise.cc:135-157, 333-366). */
void hyle_oracle_binary(int kind, int type, const void *left,
                        const int64_t *left_dims, const int64_t *left_strides,
                        int left_rank, const void *right,
                        const int64_t *right_dims,
                        const int64_t *right_strides, int right_rank, void *out,
                        const int64_t *out_dims, int out_rank);

/* Two chained Binary ops with the intermediate rounded to the storage type:
 * out = (a kind0 b) kind1 c.  All three inputs broadcast to out. This equals
 * running hyle_oracle_binary twice through a temporary. */
void hyle_oracle_binary_chain(int kind0, int kind1, int type, const void *a,
                              const int64_t *a_dims, const int64_t *a_strides,
                              int a_rank, const void *b, const int64_t *b_dims,
                              const int64_t *b_strides, int b_rank,
                              const void *c, const int64_t *c_dims,
                              const int64_t *c_strides, int c_rank, void *out,
                              const int64_t *out_dims, int out_rank);

/* src/simd/math/activations.cc:21-25,44-47 */
float hyle_oracle_sigmoid(float x);
float hyle_oracle_silu(float x);
/* src/simd/math/activations.cc:106-112 (unary_storage) */
void hyle_oracle_silu_rows(int type, const void *src, void *dst, size_t n);
/* src/simd/math/activations.cc:114-122 (gated_storage, activation = silu) */
void hyle_oracle_swiglu(int type, const void *gate, const void *value,
                        void *dst, size_t n);
/* Every UnaryKind (include/hyle/compute/operation.h:57-73: abs 0, neg 1, exp 2,
 * log 3, sqrt 4, rsqrt 5, tanh 6, sigmoid 7, relu 8, gelu 9, gelu_tanh 10,
 * silu 11, softplus 12) in the reference's scalar forms
 * (src/compute_provider_native/elementwise.cc:30-55, src/simd/math/activations.cc:21-47,
 * tests/compute_provider_native/elementwise_test.cc:43-82). */
float hyle_oracle_unary_scalar(int kind, float x);
void hyle_oracle_unary(int kind, int type, const void *src, void *dst, size_t n);
/* activation(gate) * value, activation = silu 0, gelu 1, gelu_tanh 2
 * (src/simd/math/activations.cc:114-122). */
void hyle_oracle_gated(int activation, int type, const void *gate, const void *value,
                       void *dst, size_t n);
/* GatedInputKind::kPackedHalves: row = [gate half | value half]
 * (src/compute_provider_native/elementwise.cc:192-208). */
void hyle_oracle_swiglu_packed(int type, const void *packed, void *dst,
                               size_t rows, size_t hidden);

/* ---- normalisation ------------------------------------------------------ */
/* src/simd/math/activations.cc:124-146 (fma chain, x*inv*w).  weight may be
 * NULL.  weight_type may be HYLE_ORACLE_F32 for a narrow input
 * (src/compute_ops/operation.cc:492-505). */
void hyle_oracle_rms_norm_row(int type, int weight_type, const void *src,
                              const void *weight, void *dst, size_t n,
                              float epsilon);
void hyle_oracle_rms_norm(int type, int weight_type, const void *src,
                          const void *weight, void *dst, size_t rows,
                          size_t hidden, float epsilon);
/* LayerNorm over the last axis, src/simd/math/activations.cc:148-175.  scale
 * and bias may both be NULL; with scale alone the result is normalised * scale
 * (the provider-level form of tests/compute_provider_native/normalization_test.cc:69-127,
 * which the scalar floor does not have).  param_type may be HYLE_ORACLE_F32 for
 * a narrow input. */
void hyle_oracle_layer_norm_row(int type, int param_type, const void *src,
                                const void *scale, const void *bias, void *dst,
                                size_t n, float epsilon);
void hyle_oracle_layer_norm(int type, int param_type, const void *src,
                            const void *scale, const void *bias, void *dst,
                            size_t rows, size_t hidden, float epsilon);
/* src/compute_provider_native/normalization.cc:41-80: 128-wide f32 tiles,
 * squares += dot(tile, tile); (x * inv) then * w; one RN-even store. */
void hyle_oracle_rms_norm_native(int type, int weight_type, const void *src,
                                 const void *weight, void *dst, size_t rows,
                                 size_t hidden, float epsilon);

/* ---- softmax / reductions ---------------------------------------------- */
/* src/simd/math/activations.cc:177-192,301-317.  In place allowed. */
void hyle_oracle_softmax_f32_row(const float *src, float *dst, size_t n);
/* Row softmax over the last axis of a dense [rows, width] tensor of storage
 * type `type` with `scale` and an optional broadcast mask
 * (src/compute_provider_native/transformer.cc:44-57,165-191).  The mask is
 * described by dims/byte strides and broadcast against in_dims
 * (rank in_rank, last axis = width).  mask_kind BOOLEAN: uint8 0 => -inf;
 * ADDITIVE: same storage type, v + mask
 * (src/compute_provider_cuda/reduction_kernel.cu:130-146). */
void hyle_oracle_softmax(int type, const void *src, void *dst,
                         const int64_t *in_dims, int in_rank, float scale,
                         int mask_kind, const void *mask,
                         const int64_t *mask_dims, const int64_t *mask_strides,
                         int mask_rank);

/* LogSoftmax: the same rows, masks and scale as hyle_oracle_softmax; per row
 * (v - max) - log1p(sum of exp(v - max) over every column but the first
 * maximum), NaN when the maximum is not finite
 * (src/compute_provider_cuda/reduction_kernel.cu:73-86,148-196). */
void hyle_oracle_log_softmax_f32_row(const float *src, float *dst, size_t n);
/* The same row in the scalar floor's own form (double sum, one log, one shift;
 * src/simd/math/activations.cc:320-336), pinned bit for bit against the floor
 * compiled from the reference's sources; hyle_oracle_log_softmax_f32_row is
 * held to it at the reference's bound (4e-6 relative + 2e-7). */
void hyle_oracle_log_softmax_floor_f32_row(const float *src, float *dst, size_t n);
void hyle_oracle_log_softmax(int type, const void *src, void *dst,
                             const int64_t *in_dims, int in_rank, float scale,
                             int mask_kind, const void *mask,
                             const int64_t *mask_dims, const int64_t *mask_strides,
                             int mask_rank);

/* src/compute_provider_native/reduction.cc:24-47 (NaN-propagating extrema,
 * identities +-inf) and src/compute_provider_cuda/reduction_kernel.cu:92-116
 * (sum / mean, f32 accumulate, mean of an empty row is NaN).  Reduces the
 * last axis of dense [rows, width]. */
void hyle_oracle_reduce_last_axis(int kind, int type, const void *src,
                                  void *dst, size_t rows, size_t width);

/* Reduce over the axes in `axes_mask` (bit a = axis a) of a tensor given by
 * dims and BYTE strides of any alignment; `dst` is the dense result, one
 * element per combination of the kept axes in row-major order
 * (src/compute_provider_cuda/reduction_kernel.cu:38-48, 88-113;
 * src/compute_provider_native/reduction.cc:82-111). */
void hyle_oracle_reduce(int kind, int type, const void *src, int rank,
                        const int64_t *dims, const int64_t *byte_strides,
                        uint32_t axes_mask, void *dst);

/* TopK(count = k) along `axis` of a tensor given by dims and BYTE strides:
 * numbers before NaNs, larger first (smaller first when largest == 0), equal
 * numbers and NaNs in index order; `values` holds copies of the source bits,
 * `indices` positions along the axis; both dense with the axis extent k
 * (tests/compute_route_vulkan/topk_test_support.h:62-76;
 * src/compute_ops/operation.cc:1622-1657). */
void hyle_oracle_topk(int type, const void *src, int rank, const int64_t *dims,
                      const int64_t *byte_strides, int axis, size_t k, int largest,
                      void *values, int32_t *indices);

/* include/hyle/simd/search.h:11-19: first index of the maximum; first NaN
 * index when any NaN is present; n for an empty range. */
size_t hyle_oracle_index_of_max_f32(const float *data, size_t n);
/* TopK{count=1, largest} rule: src/compute_provider_cuda/collectives.cu:478-495
 * (non-NaN beats NaN, ties -> lower index; an all-NaN row returns index 0). */
void hyle_oracle_topk1_f32(const float *data, size_t rows, size_t width,
                           float *values, int32_t *indices);

/* ---- Q8_0 --------------------------------------------------------------- */
/* Block = { fp16 d; int8 qs[32] }, 34 bytes, little-endian
 * (src/compute_ops/low_precision.cc:28-29; ggml block_q8_0, module ggml pinned
 * at ffa4e8b80930029a35991f94e7c8a93cd67730ab in cmake/HyleDependencyLock.json).
 * y = (float)qs[j] * f16_to_f32(d), stored as bf16 RN-even.  sumsq[row] is the
 * f32 sum over the exact f32 products (before bf16 rounding), accumulated in
 * index order; sumsq_rounded (optional, may be NULL) sums the squares of the
 * bf16-rounded outputs instead. */
void hyle_oracle_q8_0_dequant_bf16(const void *blocks, size_t rows, size_t k,
                                   size_t row_stride_bytes, uint16_t *out,
                                   float *sumsq, float *sumsq_rounded);
/* MatMul over a GGUF weight as the reference's ggml CPU route computes it: 8-bit
 * activation blocks (Q8_0 blocks of 32 for a Q8_0 weight, Q8_K blocks of 256 for
 * Q4_K / Q6_K), integer block dot products, f32 scales.  Restated from the
 * reference's own tests, which hold the activation codecs and the value and
 * bound they accept of the native result
 * (tests/compute_models/dspark_original_shared_reference.h:147-185,219-262;
 * tests/compute_models/qwen27_original_nextn_reference.h:74-130,144-167,193-257).
 * kind: 0 = Q4_K, 1 = Q6_K, 2 = Q8_0.  x is [m, k] f32; centre and bound are
 * [m, rows].  scales: k / 32 (Q8_0) or k / 256 (Q8_K) floats. */
void hyle_oracle_quantize_q8_0(const float *x, size_t k, int8_t *codes, float *scales);
void hyle_oracle_quantize_q8_k(const float *x, size_t k, int8_t *codes, float *scales);
void hyle_oracle_gguf_matvec_q8(int kind, const void *blocks, size_t rows, size_t k,
                                size_t row_stride_bytes, const float *x, size_t m,
                                double *centre, double *bound);
/* ggml dequantize_row_q8_0 to f32 */
/* GGUF Q4_K (kind 0: 256 elements in 144 bytes) and Q6_K (kind 1: 256 in 210)
 * rows -> f32 and / or bf16 [rows, k] plus the f32 row sums of squares of the
 * exact f32 values.  Geometry from src/compute_ops/low_precision.cc:22-27; the
 * decode is ggml's, restated from the published block layouts and pinned bit
 * for bit against the two readings of them the reference tree holds
 * (third_party/ggml_q4k_apple/ggml_q4k_apple.h:9-38;
 * tests/compute_models/qwen27_original_nextn_reference.h:74-86,262-287). */
void hyle_oracle_k_quant_dequant(int kind, const void *blocks, size_t rows, size_t k,
                                 size_t row_stride_bytes, float *out_f32, uint16_t *out_bf16,
                                 float *sumsq);

/* y[m][n] = sum_k w[n][k] * x[m][k] for GGUF rows (kind 0 Q4_K, 1 Q6_K, 2
 * Q8_0) decoded exactly, accumulated in double; `magnitude` (optional) gets
 * sum_k |w * x|.  MatMul with exact weights, not ggml's quantised-activation
 * product. */
void hyle_oracle_gguf_matvec(int kind, const void *blocks, size_t rows, size_t k,
                             size_t row_stride_bytes, const float *x, size_t m,
                             double *out, double *magnitude);

void hyle_oracle_q8_0_dequant_f32(const void *blocks, size_t rows, size_t k,
                                  size_t row_stride_bytes, float *out);

/* ---- Cast / Copy ------------------------------------------------------- */
/* Cast of a plain tensor (dims + byte strides, elements need not be aligned) to
 * a dense tensor of dst_type (src/compute_provider_native/cast.cc:73-92,225-238):
 * float <-> float decodes to f32 and encodes once (RN-even codecs above);
 * int32 -> f32 rounds to nearest even; float -> Bool is the truth of the stored
 * magnitude bits; Bool -> float is 1 or 0; equal types keep the bytes (Copy,
 * src/compute_provider_native/transform.cc:85-89).  Returns 0, or -1 for a pair
 * the reference does not define (f32 -> int32, ...). */
int hyle_oracle_cast(int src_type, int dst_type, const void *src,
                     const int64_t *dims, const int64_t *strides, int rank,
                     void *dst);

/* ---- Fill / Select ------------------------------------------------------ */
/* Storage-only members of the reference's elementwise kernel family
 * (src/compute_provider_cuda/tensor_kernel.cu:168-199): Fill writes the low
 * `width` bytes of the scalar's bits to each of n elements; Select broadcasts a
 * Bool condition and two branches of `width`-byte elements (dims + byte strides
 * each) to the dense out_dims and keeps the first branch's bytes where the
 * condition byte is non-zero, the second's elsewhere. */
void hyle_oracle_fill(size_t width, uint64_t bits, size_t n, void *dst);
void hyle_oracle_select(size_t width, const void *condition,
                        const int64_t *condition_dims, const int64_t *condition_strides, int condition_rank,
                        const void *first, const int64_t *first_dims, const int64_t *first_strides, int first_rank,
                        const void *second, const int64_t *second_dims, const int64_t *second_strides, int second_rank,
                        const int64_t *out_dims, int out_rank, void *dst);

/* ---- Concat ------------------------------------------------------------- */
/* One input of a Concat along `axis` (src/compute_ops/operation.cc:1516-1564):
 * `dims` / byte `strides` of the input, which equals the dense output's shape
 * `out_dims` except on the axis, where it starts at `offset`; elements of
 * `width` bytes are copied bit for bit. */
void hyle_oracle_concat_part(size_t width, const void *src, const int64_t *dims,
                             const int64_t *strides, int rank, int axis, int64_t offset,
                             const int64_t *out_dims, void *dst);

/* ---- Gather -------------------------------------------------------------- */
/* Gather along `axis` (src/compute_provider_native/indexing.cc:57-91,143-276):
 * source `dims` / byte `strides`, Int32 (`wide` = 0) or Int64 indices with their
 * own dims / byte strides; the dense output has the axis replaced by the shape
 * of the indices.  Returns 0, or 1 without writing when the bounds are checked
 * and an index lies outside the axis, or when the axis is empty. */
int hyle_oracle_gather(size_t width, const void *src, const int64_t *dims, const int64_t *strides, int rank,
                       int axis, const void *indices, int wide, const int64_t *index_dims,
                       const int64_t *index_strides, int index_rank, int checked, void *dst);

/* ---- RoPE ---------------------------------------------------------------- */
/* RoPE with explicit frequencies over dense data of `type` (src/compute_ggml_runtime/
 * explicit_rope.h:11-74): all arithmetic in f32, phase = frequency * f32(position).
 * positions: int32 or (`wide`) int64, [S] or (`batched`) the data's leading dimensions
 * through the sequence axis; frequencies: f32 [rotary / 2] or (`stepped`) [S, rotary / 2]. */
void hyle_oracle_rope(int type, const void *data, const int64_t *dims, int rank, int sequence_axis,
                      const void *positions, int wide, int batched, const float *frequencies, int stepped,
                      int64_t rotary, int half_split, void *dst);

/* ---- Sampling ------------------------------------------------------------ */
/* Philox4x32-10 under the reference's addressing (third_party/random123_counter/
 * philox.h:20-44): identity = key low / high, draw low / high; block `index`
 * holds words 4 * index .. 4 * index + 3 of the row's stream. */
void hyle_oracle_philox_block(const uint32_t identity[4], uint64_t index, uint32_t out[4]);
/* RandomBits (src/compute_provider_native/sampling.cc:77-88): identities U32[rows, 4]
 * -> U32[rows, word_count]. */
void hyle_oracle_random_bits(const uint32_t *identities, size_t rows, size_t word_count, uint32_t *out);
/* The uniform in (0, 1) of a row's categorical draw (sampling.cc:155-158). */
double hyle_oracle_categorical_uniform(const uint32_t identity[4]);
/* Categorical over dense [rows, width] log-weights of `type` (sampling.cc:119-215):
 * I32 indices and, when log_probabilities is not NULL, F32 scores.  Returns 0, or 1
 * without writing when a row holds NaN or +Inf or no finite element. */
int hyle_oracle_categorical(int type, const void *logits, const uint32_t *identities, size_t rows, size_t width,
                            int32_t *indices, float *log_probabilities);

/* ---- CPU baseline legs ---------------------------------------------------
 * The same arithmetic as above in the loop shapes the reference's CPU provider
 * runs (dense rows, no per-element offset walk), over a contiguous row range
 * [row_begin, row_end) so a caller can fan rows out over threads exactly as
 * parallel_for_ranges does (src/compute_provider_native/native_plan.h:74-111).
 * Used only by the benchmark's cpu_baseline timing. */
/* out = (a[r, :] + b[:]) * s: two simd-style row passes per row
 * (src/compute_provider_native/elementwise.cc:333-348, chunk = cols). */
void hyle_oracle_rows_add_row_scale_f32(const float *a, const float *b, float s,
                                        float *out, size_t cols,
                                        size_t row_begin, size_t row_end);
/* r[row, :] = bf16(r + y) via 128-wide f32 tiles
 * (src/compute_provider_native/elementwise.cc:135-147). */
void hyle_oracle_rows_add_bf16(const uint16_t *r, const uint16_t *y,
                               uint16_t *out, size_t cols, size_t row_begin,
                               size_t row_end);
void hyle_oracle_rows_swiglu_bf16(const uint16_t *gate, const uint16_t *up,
                                  uint16_t *out, size_t cols, size_t row_begin,
                                  size_t row_end);
void hyle_oracle_rows_rms_norm_bf16(const uint16_t *x, const uint16_t *w,
                                    uint16_t *out, size_t cols, float epsilon,
                                    size_t row_begin, size_t row_end);
/* rows of a [heads, seq, seq]-shaped f32 tensor flattened to [rows, cols] with a
 * Bool mask [mask_rows, cols] reused every mask_rows rows. */
void hyle_oracle_rows_softmax_bool_f32(const float *x, const uint8_t *mask,
                                       float *out, size_t cols,
                                       size_t mask_rows, size_t row_begin,
                                       size_t row_end);
void hyle_oracle_rows_topk1_f32(const float *x, float *values, int32_t *indices,
                                size_t cols, size_t row_begin, size_t row_end);
void hyle_oracle_rows_q8_0_bf16(const void *blocks, uint16_t *out, float *sumsq,
                                size_t k, size_t row_stride, size_t row_begin,
                                size_t row_end);

#ifdef __cplusplus
}
#endif
#endif /* HYLE_ORACLE_H_ */
