// Gather along one axis (include/hyle/compute/operation.h:367-370; schema
// src/compute_ops/operation.cc:616-637,1470-1489): the output is the source with the axis replaced
// by the shape of the indices, element (outer, item, inner) = source (outer, indices[item], inner).
// Storage only: elements of 1, 2, 4 or 8 bytes keep their bits.  Admission and behaviour follow
// the reference's CUDA route (src/compute_provider_cuda/collectives_provider.cc:92-125,
// collectives.cu:79-300): plain source and Int32 / Int64 indices with any byte strides, dense
// output, and for checked bounds a first dispatch that looks at every index, so that one index
// outside the axis (negative ones included) keeps every byte of the output as it was.
#include "device_common.h"
#include "kernels.h"

namespace hyle_hip {
namespace {

struct GatherIndexView {
  const unsigned char *base;
  uint32_t count;
  int32_t rank;
  uint32_t dims[kMaxRank];
  int64_t strides[kMaxRank];
};

// Dense indices are element-aligned; strided ones may sit at any byte and are read bytewise.
template <bool kWide, bool kDense>
__device__ __forceinline__ int64_t index_at(const GatherIndexView &v, uint32_t logical) {
  if constexpr (kDense) {
    if constexpr (kWide) return reinterpret_cast<const int64_t *>(v.base)[logical];
    else return reinterpret_cast<const int32_t *>(v.base)[logical];
  } else {
    int64_t offset = 0;
    uint32_t rest = logical;
    for (int a = v.rank - 1; a >= 0; --a) {
      const uint32_t extent = v.dims[a];
      offset += (int64_t)(rest % extent) * v.strides[a];
      rest /= extent;
    }
    const unsigned char *at = v.base + offset;
    uint64_t bits = 0;
#pragma unroll
    for (int b = 0; b < (kWide ? 8 : 4); ++b) bits |= (uint64_t)at[b] << (8 * b);
    return kWide ? (int64_t)bits : (int64_t)(int32_t)(uint32_t)bits;
  }
}

// Checked bounds: block b of gather_check leaves in flags[b] whether any of its indices lies
// outside [0, extent).  Every block writes its own word, so nothing has to be cleared first.
template <bool kWide, bool kDense>
__global__ __launch_bounds__(kBlockThreads) void gather_check(GatherIndexView v, uint64_t extent, uint32_t *flags) {
  int bad = 0;
  for (uint32_t i = blockIdx.x * kBlockThreads + threadIdx.x; i < v.count; i += gridDim.x * kBlockThreads) {
    const int64_t value = index_at<kWide, kDense>(v, i);
    bad |= (value < 0 || (uint64_t)value >= extent) ? 1 : 0;
  }
  bad = __syncthreads_or(bad);
  if (threadIdx.x == 0) flags[blockIdx.x] = bad ? 1u : 0u;
}

// What the moving kernels know of the check.  flags != nullptr: a dispatch of gather_check went
// first.  flags == nullptr and status != nullptr: there are few indices and every block looks at
// all of them itself before it moves anything (one dispatch instead of two; the blocks agree
// because they read the same indices).  Both nullptr: unchecked bounds.
struct GatherVerdict {
  const uint32_t *flags;
  uint32_t flag_count;  // <= kBlockThreads
  uint32_t *status;     // 0 or kStatusIndexOutOfRange after the launch, for the host
  uint64_t extent;
};

// This thread's share of the verdict: its flag word, or its share of all indices.
template <bool kWide, bool kDense>
__device__ __forceinline__ int refusals_seen(const GatherVerdict &verdict, const GatherIndexView &v) {
  int bad = 0;
  if (verdict.flags != nullptr) {
    bad = threadIdx.x < verdict.flag_count ? (int)verdict.flags[threadIdx.x] : 0;
  } else {
    // eight indices per thread at a time, their loads in flight together
    constexpr int kBatch = 8;
    for (uint32_t first = threadIdx.x; first < v.count; first += kBatch * blockDim.x) {
      int64_t value[kBatch];
#pragma unroll
      for (int j = 0; j < kBatch; ++j) {
        const uint32_t i = first + j * blockDim.x;
        value[j] = index_at<kWide, kDense>(v, i < v.count ? i : first);
      }
#pragma unroll
      for (int j = 0; j < kBatch; ++j) bad |= (value[j] < 0 || (uint64_t)value[j] >= verdict.extent) ? 1 : 0;
    }
  }
  return bad;
}
// Every block reaches the same verdict; none writes a byte of the output when an index was refused.
__device__ __forceinline__ bool block_refuses(const GatherVerdict &verdict, int bad) {
  bad = __syncthreads_or(bad);
  if (blockIdx.x == 0 && threadIdx.x == 0) *verdict.status = bad ? kStatusIndexOutOfRange : 0u;
  return bad != 0;
}
template <bool kWide, bool kDense>
__device__ __forceinline__ bool indices_refused(const GatherVerdict &verdict, const GatherIndexView &v) {
  if (verdict.status == nullptr) return false;
  return block_refuses(verdict, refusals_seen<kWide, kDense>(verdict, v));
}
// The coordinate walk has no index view of its own: it always follows a dispatch of gather_check.
__device__ __forceinline__ bool indices_refused(const GatherVerdict &verdict) {
  if (verdict.status == nullptr) return false;
  const int bad = __syncthreads_or(threadIdx.x < verdict.flag_count ? (int)verdict.flags[threadIdx.x] : 0);
  if (blockIdx.x == 0 && threadIdx.x == 0) *verdict.status = bad ? kStatusIndexOutOfRange : 0u;
  return bad != 0;
}

// A source whose elements after the axis are contiguous and whose axes before it fold into one
// pitch: the output is `rows` rows of row_units * kUnit bytes, row r = (outer, item) copied from
// source + outer * outer_pitch + indices[item] * axis_pitch.
struct GatherRows {
  const unsigned char *source;
  uint64_t outer_pitch, axis_pitch;
  uint32_t row_units, index_count, rows;
};

template <int kUnit> struct UnitWord;
template <> struct UnitWord<16> { using type = u32x4; };
template <> struct UnitWord<8> { using type = uint64_t; };
template <> struct UnitWord<4> { using type = uint32_t; };
template <> struct UnitWord<2> { using type = uint16_t; };
template <> struct UnitWord<1> { using type = unsigned char; };

template <int kUnit> __device__ __forceinline__ typename UnitWord<kUnit>::type load_unit(const unsigned char *from, uint32_t u) {
  // plain loads: the rows of a table are picked again and again (14.0 us with the non-temporal hint
  // against 12.5 us without, for 8192 rows of 4 KiB out of 622 MB)
  if constexpr (kUnit == 16) return load16(from, u);
  else return reinterpret_cast<const typename UnitWord<kUnit>::type *>(from)[u];
}
template <int kUnit> __device__ __forceinline__ void store_unit(unsigned char *to, uint32_t u, typename UnitWord<kUnit>::type word) {
  if constexpr (kUnit == 16) store16_stream(to, u, word);
  else reinterpret_cast<typename UnitWord<kUnit>::type *>(to)[u] = word;
}

// Rows of at least 256 units, fewer than 4096 chunks in all: a row is cut into chunks of 256 units
// and a block of 512 threads takes two consecutive chunks -- of one long row or of two short ones --, one unit per thread, so
// a chunk's row, its index and both addresses are the same for 256 threads.  Measured on MI355X
// for 8192 rows of 4 KiB picked at random from 622 MB: 12.5 us in this form (11.4 us when the
// picked rows are consecutive, 11.1 us for a plain copy of the same bytes); blocks that take 4 to
// 16 chunks with their indices fetched first and their loads in flight together or one after
// another take 12.6 to 18.4 us.
constexpr int kRowThreads = 2 * kBlockThreads;
template <int kUnit, bool kWide, bool kDense>
__global__ __launch_bounds__(kRowThreads) void gather_rows(GatherRows p, GatherIndexView v, GatherVerdict verdict,
                                                           unsigned char *out, uint32_t chunks_per_row, uint32_t chunks) {
  if (indices_refused<kWide, kDense>(verdict, v)) return;
  const uint32_t chunk = blockIdx.x * (kRowThreads / kBlockThreads) + threadIdx.x / kBlockThreads;
  if (chunk >= chunks) return;
  const uint32_t row = chunk / chunks_per_row, piece = chunk - row * chunks_per_row;
  const uint32_t unit = piece * kBlockThreads + threadIdx.x % kBlockThreads;
  if (unit >= p.row_units) return;
  const uint32_t outer = row / p.index_count, item = row - outer * p.index_count;
  const int64_t selected = index_at<kWide, kDense>(v, item);
  const unsigned char *from = p.source + (uint64_t)outer * p.outer_pitch + (uint64_t)selected * p.axis_pitch;
  store_unit<kUnit>(out + (uint64_t)row * p.row_units * kUnit, unit, load_unit<kUnit>(from, unit));
}

// The same chunks, sixteen per block of 512 threads: sixteen threads resolve the chunks' rows and
// indices into LDS first, then every lane streams eight units one after another, its stores
// after its last load, as the plain copy kernel does.
constexpr int kFatChunks = 16;
template <int kUnit, bool kWide, bool kDense>
__global__ __launch_bounds__(kRowThreads) void gather_rows_fat(GatherRows p, GatherIndexView v, GatherVerdict verdict,
                                                               unsigned char *out, uint32_t chunks_per_row, uint32_t chunks) {
  __shared__ const unsigned char *from_of[kFatChunks];
  __shared__ unsigned char *to_of[kFatChunks];
  __shared__ uint32_t units_of[kFatChunks];
  // A block that checks the indices itself does so while its rows are on their way: it reads from
  // where its own indices point, held inside the axis, and stores only after the verdict.
  const bool checks_itself = verdict.status != nullptr && verdict.flags == nullptr;
  if (!checks_itself && indices_refused<kWide, kDense>(verdict, v)) return;
  if (threadIdx.x < kFatChunks) {
    const uint32_t chunk = blockIdx.x * kFatChunks + threadIdx.x;
    uint32_t units = 0;
    // a chunk past the last one (the last block's, when the chunks are no multiple of sixteen) has no
    // units, but every lane still reads "its first unit": give it an address that exists
    from_of[threadIdx.x] = p.source;
    to_of[threadIdx.x] = out;
    if (chunk < chunks) {
      const uint32_t row = chunk / chunks_per_row, piece = chunk - row * chunks_per_row;
      const uint32_t outer = row / p.index_count, item = row - outer * p.index_count;
      int64_t selected = index_at<kWide, kDense>(v, item);
      if (checks_itself) selected = selected < 0 ? 0 : ((uint64_t)selected >= verdict.extent ? (int64_t)verdict.extent - 1 : selected);
      const uint32_t first = piece * kBlockThreads;
      units = p.row_units - first < (uint32_t)kBlockThreads ? p.row_units - first : (uint32_t)kBlockThreads;
      from_of[threadIdx.x] = p.source + (uint64_t)outer * p.outer_pitch + (uint64_t)selected * p.axis_pitch + (size_t)first * kUnit;
      to_of[threadIdx.x] = out + ((uint64_t)row * p.row_units + first) * kUnit;
    }
    units_of[threadIdx.x] = units;
  }
  __syncthreads();
  constexpr int kSteps = kFatChunks * kBlockThreads / kRowThreads;  // 8
  const uint32_t lane = threadIdx.x % kBlockThreads, half = threadIdx.x / kBlockThreads;
  typename UnitWord<kUnit>::type held[kSteps];
  bool live[kSteps];
  auto load = [&](int j) {
    const int c = j * (kRowThreads / kBlockThreads) + half;
    live[j] = lane < units_of[c];
    held[j] = load_unit<kUnit>(from_of[c], live[j] ? lane : 0u);  // a lane past the chunk reads its first unit and drops it
  };
  load(0);
#pragma unroll
  for (int j = 0; j < kSteps; ++j) {
    if constexpr (kUnit == 16) loads_issued(held[j]);
    if (j + 1 < kSteps) load(j + 1);
  }
  if (checks_itself && block_refuses(verdict, refusals_seen<kWide, kDense>(verdict, v))) return;
#pragma unroll
  for (int j = 0; j < kSteps; ++j) {
    const int c = j * (kRowThreads / kBlockThreads) + half;
    if (live[j]) store_unit<kUnit>(to_of[c], lane, held[j]);
  }
}

// Short rows: one unit per thread, rows packed into blocks.
template <int kUnit, bool kWide, bool kDense>
__global__ __launch_bounds__(kBlockThreads) void gather_units(GatherRows p, GatherIndexView v, GatherVerdict verdict,
                                                              unsigned char *out, uint32_t units) {
  if (indices_refused<kWide, kDense>(verdict, v)) return;
  const uint32_t g = blockIdx.x * kBlockThreads + threadIdx.x;
  if (g >= units) return;
  const uint32_t row = g / p.row_units, u = g - row * p.row_units;
  const uint32_t outer = row / p.index_count, item = row - outer * p.index_count;
  const int64_t selected = index_at<kWide, kDense>(v, item);
  const unsigned char *from = p.source + (uint64_t)outer * p.outer_pitch + (uint64_t)selected * p.axis_pitch;
  store_unit<kUnit>(out + (uint64_t)row * p.row_units * kUnit, u, load_unit<kUnit>(from, u));
}

// Any strides: one output element per thread, walked by output coordinate.  On the axes the
// indices span source_strides is 0, elsewhere index_strides is 0.
struct GatherLayout {
  const unsigned char *source, *indices;
  int32_t rank;
  uint32_t dims[kMaxRank];
  int64_t source_strides[kMaxRank], index_strides[kMaxRank];
  int64_t axis_stride;
};

template <int kSize, bool kWide>
__global__ __launch_bounds__(kBlockThreads) void gather_general(GatherLayout l, GatherVerdict verdict, unsigned char *out,
                                                                uint64_t elements) {
  if (indices_refused(verdict)) return;
  const uint64_t e = (uint64_t)blockIdx.x * kBlockThreads + threadIdx.x;
  if (e >= elements) return;
  uint64_t rest = e;
  int64_t from = 0, index_offset = 0;
  for (int a = l.rank - 1; a >= 0; --a) {
    const uint32_t extent = l.dims[a];
    const int64_t c = (int64_t)(rest % extent);
    rest /= extent;
    from += c * l.source_strides[a];
    index_offset += c * l.index_strides[a];
  }
  const unsigned char *at = l.indices + index_offset;
  uint64_t bits = 0;
#pragma unroll
  for (int b = 0; b < (kWide ? 8 : 4); ++b) bits |= (uint64_t)at[b] << (8 * b);
  const int64_t selected = kWide ? (int64_t)bits : (int64_t)(int32_t)(uint32_t)bits;
  const unsigned char *source = l.source + from + selected * l.axis_stride;
#pragma unroll
  for (int b = 0; b < kSize; ++b) out[e * kSize + b] = source[b];
}

// Launch-shape labels: gather_<form>/<unit bytes>/<index width>/<dense|strided indices>
inline std::string index_words(bool wide, bool dense) { return std::string(wide ? "i64" : "i32") + (dense ? "/dense" : "/strided"); }
template <int kForm, int kUnit, bool kWide, bool kDense> struct GatherRowsTag {  // 0 fat rows, 1 rows, 2 units
  static std::string text() {
    return std::string(kForm == 0 ? "gather_rows_fat/" : (kForm == 1 ? "gather_rows/" : "gather_units/")) + std::to_string(kUnit) + "-bytes/" + index_words(kWide, kDense);
  }
};
template <int kSize, bool kWide> struct GatherGeneralTag {
  static std::string text() { return "gather_general/" + std::to_string(kSize) + "-bytes/" + (kWide ? "i64" : "i32"); }
};
template <bool kWide, bool kDense> struct GatherCheckTag {
  static std::string text() { return "gather_check/" + index_words(kWide, kDense); }
};

template <int kUnit, bool kWide, bool kDense>
void run_rows(const GatherRows &rows, const GatherIndexView &view, const GatherVerdict &verdict, unsigned char *out,
              hipStream_t stream) {
  const dim3 block(kBlockThreads);
  if (rows.row_units >= kBlockThreads) {
    const uint32_t per_row = (rows.row_units + kBlockThreads - 1) / kBlockThreads;
    const uint64_t chunks = (uint64_t)per_row * rows.rows;  // at most INT32_MAX bytes / 256
    const uint32_t per_block = kRowThreads / kBlockThreads;
    // Enough chunks to give every compute unit a fat block: sixteen chunks per block, resolved
    // first and then streamed (11.8 us against 12.6 us for 8192 rows of 4 KiB picked at random).
    if (chunks >= 4096) {
      note_variant<GatherRowsTag<0, kUnit, kWide, kDense>>();
      hipLaunchKernelGGL((gather_rows_fat<kUnit, kWide, kDense>), dim3((uint32_t)((chunks + kFatChunks - 1) / kFatChunks)),
                         dim3(kRowThreads), 0, stream, rows, view, verdict, out, per_row, (uint32_t)chunks);
    } else {
      note_variant<GatherRowsTag<1, kUnit, kWide, kDense>>();
      hipLaunchKernelGGL((gather_rows<kUnit, kWide, kDense>), dim3((uint32_t)((chunks + per_block - 1) / per_block)),
                         dim3(kRowThreads), 0, stream, rows, view, verdict, out, per_row, (uint32_t)chunks);
    }
  } else {
    const uint64_t units = (uint64_t)rows.rows * rows.row_units;
    note_variant<GatherRowsTag<2, kUnit, kWide, kDense>>();
    hipLaunchKernelGGL((gather_units<kUnit, kWide, kDense>), dim3((uint32_t)((units + kBlockThreads - 1) / kBlockThreads)),
                       block, 0, stream, rows, view, verdict, out, (uint32_t)units);
  }
}

template <int kUnit>
void run_rows_indexed(bool wide, bool dense, const GatherRows &rows, const GatherIndexView &view,
                      const GatherVerdict &verdict, unsigned char *out, hipStream_t stream) {
  if (wide) {
    if (dense) run_rows<kUnit, true, true>(rows, view, verdict, out, stream);
    else run_rows<kUnit, true, false>(rows, view, verdict, out, stream);
  } else {
    if (dense) run_rows<kUnit, false, true>(rows, view, verdict, out, stream);
    else run_rows<kUnit, false, false>(rows, view, verdict, out, stream);
  }
}

template <int kSize>
void run_general(bool wide, const GatherLayout &l, const GatherVerdict &verdict, unsigned char *out, uint64_t elements,
                 hipStream_t stream) {
  const dim3 grid((uint32_t)((elements + kBlockThreads - 1) / kBlockThreads)), block(kBlockThreads);
  if (wide) {
    note_variant<GatherGeneralTag<kSize, true>>();
    hipLaunchKernelGGL((gather_general<kSize, true>), grid, block, 0, stream, l, verdict, out, elements);
  } else {
    note_variant<GatherGeneralTag<kSize, false>>();
    hipLaunchKernelGGL((gather_general<kSize, false>), grid, block, 0, stream, l, verdict, out, elements);
  }
}

}  // namespace

hipError_t launch_gather(const GatherParams &p, const void *source, const void *indices, void *out, void *workspace,
                         hipStream_t stream) {
  if (p.elements == 0) return hipSuccess;
  GatherIndexView view{};
  view.base = static_cast<const unsigned char *>(indices);
  view.count = p.index_count;
  view.rank = p.index_rank;
  for (int a = 0; a < kMaxRank; ++a) {
    view.dims[a] = p.index_dims[a];
    view.strides[a] = p.index_strides[a];
  }
  // strided indices are read bytewise; dense ones at their natural alignment
  const bool dense_indices = p.dense_indices && reinterpret_cast<uintptr_t>(indices) % (p.wide_indices ? 8 : 4) == 0;
  GatherVerdict verdict{nullptr, 0, nullptr, p.extent};
  if (p.checked && p.fused_check) {
    verdict.status = static_cast<uint32_t *>(workspace) + kGatherStatusWord;
  } else if (p.checked) {
    uint32_t *words = static_cast<uint32_t *>(workspace);
    const uint32_t blocks = std::min<uint32_t>(kBlockThreads, (p.index_count + kBlockThreads - 1) / kBlockThreads);
    verdict = GatherVerdict{words, blocks, words + kGatherStatusWord, p.extent};
    const dim3 grid(blocks), block(kBlockThreads);
    if (p.wide_indices) {
      if (dense_indices) { note_variant<GatherCheckTag<true, true>>(); hipLaunchKernelGGL((gather_check<true, true>), grid, block, 0, stream, view, p.extent, words); }
      else { note_variant<GatherCheckTag<true, false>>(); hipLaunchKernelGGL((gather_check<true, false>), grid, block, 0, stream, view, p.extent, words); }
    } else {
      if (dense_indices) { note_variant<GatherCheckTag<false, true>>(); hipLaunchKernelGGL((gather_check<false, true>), grid, block, 0, stream, view, p.extent, words); }
      else { note_variant<GatherCheckTag<false, false>>(); hipLaunchKernelGGL((gather_check<false, false>), grid, block, 0, stream, view, p.extent, words); }
    }
    const hipError_t err = hipGetLastError();
    if (err != hipSuccess) return err;
  }
  unsigned char *o = static_cast<unsigned char *>(out);
  if (p.rows) {
    // the widest unit that divides the row, both pitches and both addresses
    const uint64_t row_bytes = p.inner * p.size;
    uint64_t together = row_bytes | reinterpret_cast<uintptr_t>(source) | reinterpret_cast<uintptr_t>(out);
    if (p.extent > 1) together |= p.axis_pitch;
    if (p.outer > 1) together |= p.outer_pitch;
    int unit = 16;
    while (together % unit != 0) unit /= 2;
    GatherRows rows{static_cast<const unsigned char *>(source), p.outer_pitch, p.axis_pitch, (uint32_t)(row_bytes / unit),
                    p.index_count, p.outer * p.index_count};
    switch (unit) {
      case 16: run_rows_indexed<16>(p.wide_indices, dense_indices, rows, view, verdict, o, stream); break;
      case 8: run_rows_indexed<8>(p.wide_indices, dense_indices, rows, view, verdict, o, stream); break;
      case 4: run_rows_indexed<4>(p.wide_indices, dense_indices, rows, view, verdict, o, stream); break;
      case 2: run_rows_indexed<2>(p.wide_indices, dense_indices, rows, view, verdict, o, stream); break;
      default: run_rows_indexed<1>(p.wide_indices, dense_indices, rows, view, verdict, o, stream); break;
    }
    return hipGetLastError();
  }
  GatherLayout l{};
  l.source = static_cast<const unsigned char *>(source);
  l.indices = view.base;
  l.rank = p.rank;
  l.axis_stride = (int64_t)p.axis_pitch;
  for (int a = 0; a < kMaxRank; ++a) {
    l.dims[a] = p.dims[a];
    l.source_strides[a] = p.source_strides[a];
    l.index_strides[a] = p.index_out_strides[a];
  }
  switch (p.size) {
    case 8: run_general<8>(p.wide_indices, l, verdict, o, p.elements, stream); break;
    case 4: run_general<4>(p.wide_indices, l, verdict, o, p.elements, stream); break;
    case 2: run_general<2>(p.wide_indices, l, verdict, o, p.elements, stream); break;
    default: run_general<1>(p.wide_indices, l, verdict, o, p.elements, stream); break;
  }
  return hipGetLastError();
}

}  // namespace hyle_hip
