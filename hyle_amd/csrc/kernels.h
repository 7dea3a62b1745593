// kernels.h -- host-callable launchers of the gfx950 kernels.  Each launcher
// only enqueues on the given stream; shapes were validated when the plan was
// built, pointer alignment is checked by the caller at launch time.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <string>

namespace hyle_hip {

// ---- launch-shape labels ------------------------------------------------------
// Which kernel shape a launcher picks depends on sizes, strides and alignment seen at launch.
// Every launcher notes a label for the shape it chose on the calling thread, and every label
// registers itself when the library loads, so the list (hyle_hip_variant_label) holds exactly
// the launch shapes compiled in.  A label names the shape (lanes x vectors x rows, mask form,
// exact or masked), not the storage type: tests use it to prove that a case reached the kernel
// it was written for.
namespace variants {
const char *add(const std::string &label);  // registers a label, returns its stable text
void note(const char *label);               // the calling thread is about to launch this shape
}  // namespace variants

// Tag::text() is the label; the first use of Variant<Tag>::label anywhere in the library makes
// the label part of the list.
template <class Tag> struct Variant {
  static const char *const label;
};
template <class Tag> const char *const Variant<Tag>::label = variants::add(Tag::text());
template <class Tag> inline void note_variant() { variants::note(Variant<Tag>::label); }

enum class Elem : uint8_t { kF32 = 0, kF16 = 1, kBF16 = 2 };

inline int elem_size(Elem e) { return e == Elem::kF32 ? 4 : 2; }
inline int elem_vec(Elem e) { return e == Elem::kF32 ? 4 : 8; }

constexpr int kMaxRank = 8;

// ---- elementwise ------------------------------------------------------------
// kUnary: kind0 = UnaryKind; kGated: kind0 = GatedActivationKind (kSilu / kSwiglu are the SiLU forms)
enum class EwOp : uint8_t { kBinary = 0, kChain, kSilu, kSwiglu, kUnary, kGated };

// How one input is addressed by the flat (vectorised) kernel: every `period`
// elements the operand repeats (0 = never, the operand is as large as the
// output); period 1 is a scalar splat.
struct EwFlat {
  uint64_t elements = 0;      // output elements
  uint32_t period[3] = {0, 0, 0};
  EwOp op = EwOp::kBinary;
  uint8_t kind0 = 0, kind1 = 0;
  uint8_t inputs = 2;
};

// Fully general addressing: dense output of `rank` dims, per-input byte strides
// (0 on broadcast axes).
struct EwGeneral {
  uint64_t elements = 0;
  int32_t rank = 0;
  uint32_t dims[kMaxRank] = {};
  int64_t strides[3][kMaxRank] = {};
  EwOp op = EwOp::kBinary;
  uint8_t kind0 = 0, kind1 = 0;
  uint8_t inputs = 2;
};

// Packed SwiGLU: rows of [gate | value], each `hidden` wide.
struct EwPacked {
  uint64_t rows = 0;
  uint32_t hidden = 0;
  uint8_t activation = 0;  // GatedActivationKind
};

hipError_t launch_ew_flat(Elem type, const EwFlat &p, const void *a, const void *b, const void *c,
                          void *out, bool vectorised, hipStream_t stream);
hipError_t launch_ew_general(Elem type, const EwGeneral &p, const void *a, const void *b,
                             const void *c, void *out, hipStream_t stream);
hipError_t launch_swiglu_packed(Elem type, const EwPacked &p, const void *packed, void *out,
                                bool vectorised, hipStream_t stream);

// ---- row kernels ------------------------------------------------------------
struct RowShape {
  uint64_t rows = 0;
  uint32_t width = 0;
};

struct NormParams {
  RowShape shape;
  float epsilon = 0;
  bool has_weight = false;
  bool weight_f32 = false;  // f32 parameters with a narrow input
  bool layer = false;       // LayerNorm: subtract the row mean first
  bool has_bias = false;    // LayerNorm only, together with a weight
};
hipError_t launch_norm(Elem type, const NormParams &p, const void *x, const void *w, const void *b,
                       void *y, bool vectorised, hipStream_t stream);

// Softmax over the last axis of a dense [rows, width] tensor.  The mask row of
// logical row r starts at mask + sum_k coord_k(r) * outer_stride[k]; inside the
// row the mask advances by `mask_inner_stride` bytes per column (0 = one value
// for the whole row).
struct SoftmaxParams {
  RowShape shape;
  float scale = 1.0f;
  uint8_t mask_kind = 0;  // HYLE_HIP_MASK_*
  bool log = false;
  int32_t outer_rank = 0;
  uint32_t outer_dims[kMaxRank] = {};
  int64_t mask_outer_strides[kMaxRank] = {};
  int64_t mask_inner_stride = 0;
};
hipError_t launch_softmax(Elem type, const SoftmaxParams &p, const void *x, const void *mask,
                          void *y, bool vectorised, int compute_units, hipStream_t stream);

// Softmax along any axis of a strided tensor: rows = outer * inner.
struct SoftmaxGeneralParams {
  uint64_t outer = 0, inner = 0;
  uint32_t width = 0;
  float scale = 1.0f;
  uint8_t mask_kind = 0;
  bool log = false;
  int32_t rank = 0;
  int32_t axis = 0;
  uint32_t dims[kMaxRank] = {};
  int64_t in_strides[kMaxRank] = {};
  int64_t mask_strides[kMaxRank] = {};
};
hipError_t launch_softmax_general(Elem type, const SoftmaxGeneralParams &p, const void *x,
                                  const void *mask, void *y, hipStream_t stream);

// Reduce over a set of axes.  rows = results, width = elements folded into each result.
enum class ReduceForm : uint8_t {
  kRows,     // dense, reduced axes innermost: [rows, width]
  kColumns,  // dense [outer, reduced, inner], inner > 1
  kGeneral,  // byte strides and any set of axes
};
struct ReduceParams {
  uint8_t kind = 0;  // HYLE_HIP_REDUCE_*
  ReduceForm form = ReduceForm::kGeneral;
  uint32_t rows = 0, width = 0;
  float divisor = 1.0f;  // the mean's count (0 for an empty reduction: the mean is NaN)
  uint32_t outer = 1, reduced = 1, inner = 1;  // kColumns
  // set by reduce_plan
  uint32_t tiles = 1, tile_width = 0;          // kRows: pieces of one row
  uint32_t segments = 1, segment_rows = 0;     // kColumns: pieces of the reduced extent
  size_t workspace_bytes = 0;                  // f32 partial results of a two-dispatch launch
  uint32_t dispatches = 1;
  // kGeneral
  int32_t rank = 0;
  uint32_t axes = 0;  // bit a: axis a is reduced
  uint32_t dims[kMaxRank] = {};
  int64_t strides[kMaxRank] = {};
  bool bytewise = false;  // strides or addresses that are not multiples of the element size
};
void reduce_plan(Elem type, ReduceParams *p);
hipError_t launch_reduce(Elem type, const ReduceParams &p, const void *x, void *y, void *workspace,
                         bool input_vector_aligned, hipStream_t stream);

// TopK(count = 1): a scan dispatch leaves per-tile candidates in the workspace, a fold dispatch
// turns them into the outputs.
struct ArgmaxParams {
  RowShape shape;
  uint32_t tiles = 0;        // tiles per row
  uint32_t tile_elems = 0;   // elements per tile
};
void argmax_plan(uint64_t rows, uint32_t width, Elem type, uint32_t compute_units, ArgmaxParams *p);
size_t argmax_workspace_bytes(const ArgmaxParams &p);
hipError_t launch_argmax(Elem type, const ArgmaxParams &p, const void *x, void *values,
                         int32_t *indices, void *workspace, bool vectorised, hipStream_t stream);

// TopK(count = k) along any axis of a plain tensor: sorted tiles, then merges of k-key lists
// through the workspace.
struct TopKParams {
  uint32_t rows = 0, width = 0, count = 0, inner = 1;
  bool largest = true;
  bool dense_last = false;  // dense tensor, axis innermost
  bool bytewise = false;    // strides that are not multiples of the element size
  bool integer = false;     // int32 elements (the Elem passed to launch_topk is then ignored)
  int32_t rank = 0, axis = 0;
  uint32_t dims[kMaxRank] = {};
  int64_t strides[kMaxRank] = {};
  // set by topk_plan
  bool select = false;           // count small enough for the register-resident selection
  bool runs = false;             // count above 1024: whole sorted tiles merged as runs, two at a time
  uint32_t tile_elements = 0;    // elements of a row one block of the first dispatch takes
  uint32_t tiles = 1, fan = 2, dispatches = 1;
  size_t workspace_bytes = 0;
};
uint32_t topk_max_count();
void topk_plan(TopKParams *p);
hipError_t launch_topk(Elem type, const TopKParams &p, const void *x, void *values, int32_t *indices,
                       void *workspace, bool input_vector_aligned, hipStream_t stream);

// GGUF Q4_K (kind 0, 144-byte blocks) / Q6_K (kind 1, 210-byte blocks) rows of k/256 blocks
// -> bf16 [rows, k] + f32 sumsq[rows].
struct KQuantParams {
  uint64_t rows = 0;
  uint32_t k = 0;
  uint64_t row_stride = 0;  // bytes between physical rows
  uint8_t kind = 0;
};
hipError_t launch_k_quant_dequant(const KQuantParams &p, const void *blocks, void *out, float *sumsq,
                                  hipStream_t stream);

// y[m][n] = sum_k w[n][k] * x[m][k], w a GGUF weight (kind 0 Q4_K, 1 Q6_K, 2 Q8_0), x [m, k] dense.
struct MatVecParams {
  uint64_t rows = 0;        // N
  uint32_t k = 0, m = 0;
  uint64_t row_stride = 0;  // bytes between physical weight rows
  uint8_t kind = 0;
  uint8_t codec = 0;        // HYLE_HIP_ACTIVATIONS_*: 0 exact f32 activations, 1 ggml's 8-bit activation blocks
  uint32_t compute_units = 256;  // of the plan's device: the grids are three blocks per unit
};
size_t gguf_matvec_shared_bytes(uint32_t m, uint32_t k);
// The 8-bit activation route: any whole number of blocks per row at even addresses, M <= 8.
// Rows of 2048 n values made of whole 16-byte vectors take the span kernels (the codes of all M
// rows in LDS: gguf_matvec_q8_shared_bytes); other shapes walk block by block, M in groups that
// fit LDS (gguf_matvec_q8_dispatches launches).  gguf_matvec_q8_serves: one activation row fits.
size_t gguf_matvec_q8_shared_bytes(uint32_t m, uint32_t k);
bool gguf_matvec_q8_serves(int kind, uint32_t k);
uint32_t gguf_matvec_q8_dispatches(int kind, uint32_t m, uint32_t k, uint64_t row_stride);
hipError_t launch_gguf_matvec_q8(Elem x_type, const MatVecParams &p, const void *weights, const void *x, void *y,
                                 int compute_units, hipStream_t stream);
hipError_t launch_gguf_matvec(Elem x_type, const MatVecParams &p, const void *weights, const void *x, void *y,
                              hipStream_t stream);

// Q8_0 rows of k/32 blocks {f16 d; int8 qs[32]} -> bf16 [rows, k] + f32 sumsq[rows].
struct Q8Params {
  uint64_t rows = 0;
  uint32_t k = 0;
  uint64_t row_stride = 0;  // bytes between physical rows
};
hipError_t launch_q8_0_dequant(const Q8Params &p, const void *blocks, void *out, float *sumsq,
                               bool vectorised, hipStream_t stream);

// Cast between storage types, or Copy (copy_size = element bytes, types ignored): any plain
// input (dims + byte strides, elements need not be aligned) to a dense output.
enum class CastType : uint8_t { kF32 = 0, kF16, kBF16, kBool, kI32 };
struct CastParams {
  uint64_t elements = 0;
  CastType src = CastType::kF32, dst = CastType::kF32;
  uint8_t copy_size = 0;     // 0: convert; 1, 2, 4: move elements of that size unchanged
  bool dense_input = false;  // the input is dense too: the flat kernels apply
  int32_t rank = 0;
  uint32_t dims[kMaxRank] = {};
  int64_t strides[kMaxRank] = {};  // input byte strides
};
hipError_t launch_cast(const CastParams &p, const void *in, void *out, bool vectorised,
                       hipStream_t stream);

// Fill: `elements` elements of `size` bytes (1, 2, 4 or 8) set to the low bytes of `bits`.
struct FillParams {
  uint64_t elements = 0;
  uint64_t bits = 0;
  uint8_t size = 4;
};
hipError_t launch_fill(const FillParams &p, void *out, hipStream_t stream);

// Select(condition Bool, first, second) -> dense output of `size`-byte elements.  flat: every
// operand is dense and either as long as the output or one element (scalar[i]); otherwise byte
// strides per output axis (0 where an operand is broadcast).
struct SelectParams {
  uint64_t elements = 0;
  uint8_t size = 4;
  bool flat = false;
  bool scalar[3] = {false, false, false};
  int32_t rank = 0;
  uint32_t dims[kMaxRank] = {};
  int64_t strides[3][kMaxRank] = {};
};
hipError_t launch_select(const SelectParams &p, const void *condition, const void *first, const void *second, void *out,
                         bool vector_aligned, hipStream_t stream);

// Concat of `inputs` (1..4) plain tensors along `axis` into a dense output seen as [outer, total,
// inner]; input i covers [offset[i], offset[i] + extent[i]) of the axis.  dense: every input is
// dense (runs of extent * inner elements are contiguous), otherwise byte strides per input.
struct ConcatParams {
  uint64_t elements = 0;   // of the output
  uint32_t inputs = 0, outer = 1, inner = 1, total = 0;
  uint32_t extent[4] = {}, offset[4] = {};
  uint8_t size = 4;
  bool dense = true;
  int32_t rank = 0, axis = 0;
  uint32_t dims[kMaxRank] = {};
  int64_t strides[4][kMaxRank] = {};
};
hipError_t launch_concat(const ConcatParams &p, const void *const *inputs, void *out, hipStream_t stream);

// Gather along one axis of a plain source by Int32 / Int64 indices into a dense output seen as
// [outer, index_count, inner].  rows: the elements after the axis are contiguous and the axes
// before it fold into outer_pitch, so whole rows move; otherwise the output is walked by
// coordinate with source_strides / index_out_strides per output axis.  checked: a first dispatch
// leaves one flag per block in the workspace (32-bit words from its start) and the moving dispatch
// writes nothing when any is set -- or, with few indices, every moving block checks them all
// itself; word kGatherStatusWord then reads 1, else 0.
constexpr uint32_t kGatherStatusWord = 256;
constexpr size_t kGatherWorkspaceBytes = (kGatherStatusWord + 1) * 4;
struct GatherParams {
  uint64_t elements = 0;  // of the output
  uint64_t extent = 0;    // of the source on the axis
  uint64_t inner = 1;     // elements after the axis
  uint64_t outer_pitch = 0, axis_pitch = 0;  // bytes
  uint32_t outer = 1, index_count = 0;
  uint8_t size = 4;
  bool wide_indices = false, dense_indices = true, checked = true, rows = false;
  bool fused_check = false;  // checked, whole rows, few indices or a large launch: every moving block looks at all indices itself
  int32_t index_rank = 0;
  uint32_t index_dims[kMaxRank] = {};
  int64_t index_strides[kMaxRank] = {};
  int32_t rank = 0;  // of the output
  uint32_t dims[kMaxRank] = {};
  int64_t source_strides[kMaxRank] = {}, index_out_strides[kMaxRank] = {};
};
hipError_t launch_gather(const GatherParams &p, const void *source, const void *indices, void *out, void *workspace,
                         hipStream_t stream);

// RoPE over a dense tensor seen as `rows` rows of `depth` elements; row r belongs to sequence step
// (r / inner) % sequence.  Positions are [sequence] or, batched, one per (r / inner); frequencies
// are f32 [rotary / 2] or, stepped, [sequence, rotary / 2].
struct RopeParams {
  uint64_t rows = 0;
  uint32_t depth = 0, rotary = 0, sequence = 1, inner = 1;
  bool half_split = false, wide_positions = false, batched_positions = false, stepped_frequencies = false;
};
hipError_t launch_rope(Elem type, const RopeParams &p, const void *in, const void *positions, const void *frequencies, void *out,
                       bool vector_aligned, hipStream_t stream);

// What a status word in the workspace says after a launch whose kernels can refuse their input
// (the reference's DeviceStatusCode): 0 accepted.
constexpr uint32_t kStatusIndexOutOfRange = 1, kStatusInvalidNumericInput = 2;

// RandomBits: U32[rows, 4] identities -> U32[rows, word_count] Philox4x32-10 words.
struct RandomBitsParams {
  uint32_t rows = 0, word_count = 0;
};
hipError_t launch_random_bits(const RandomBitsParams &p, const void *identities, void *out, hipStream_t stream);

// Categorical over dense [rows, width] log-weights: `tiles` tiles of kCategoricalTile elements per
// row, one CategoricalTile each at the start of the workspace, the status word at status_offset.
constexpr int kCategoricalTile = 4096;
struct CategoricalTile {
  float maximum;     // of the tile (-inf: no finite element)
  uint32_t invalid;  // the tile holds NaN or +inf
  double mass;       // sum of exp(x - maximum)
};
struct CategoricalParams {
  uint32_t rows = 0, width = 0, tiles = 0;
  bool scored = false;  // also the selected element's normalised log probability
  size_t status_offset = 0;
};
hipError_t launch_categorical(Elem type, const CategoricalParams &p, const void *logits, const void *identities, void *indices,
                              void *scores, void *workspace, bool vector_aligned, hipStream_t stream);

}  // namespace hyle_hip
