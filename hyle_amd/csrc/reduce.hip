// Reduce (sum, mean, minimum, maximum) over any set of axes.
//
// Semantics follow the reference's CUDA provider (src/compute_provider_cuda/reduction_kernel.cu:
// 38-48 coordinates, 62-71 NaN-propagating extrema, 88-113 one result per output element,
// f32 accumulation, mean = sum / count with NaN for an empty reduction) and its schema
// (src/compute_ops/operation.cc:1345-1392).  Sums may be taken in any order
// (include/hyle/compute/operation.h:314-318 allows reassociation for f32).
//
// Three memory shapes, chosen when the plan is made:
//   rows     the reduced axes are the innermost ones of a dense tensor: [rows, width], a row is
//            contiguous.  A wave or a block per row; few long rows are cut into tiles whose
//            f32 partial results go through the caller's workspace to a second, tiny dispatch
//            (one compute unit streams only ~35 GB/s, so a lone row must be spread out).
//   columns  a dense tensor seen as [outer, reduced, inner] with inner > 1: lanes lie along
//            `inner` (16-byte vectors, coalesced), the rows of `reduced` are shared out over
//            the rest of the block and, when there are too few blocks, over grid segments
//            that meet in the workspace.
//   general  anything else (strides, scattered axes, unaligned bytes): one wave per result,
//            coordinates by division.  Correct, not tuned.
#include <algorithm>

#include "device_common.h"
#include "kernels.h"

namespace hyle_hip {
namespace {

enum : int { kSum = 0, kMean = 1, kMinimum = 2, kMaximum = 3 };

template <int kKind> __device__ __forceinline__ float reduce_identity() {
  return kKind == kMinimum ? INFINITY : kKind == kMaximum ? -INFINITY : 0.0f;
}
template <int kKind> __device__ __forceinline__ float reduce_step(float acc, float v) {
  if constexpr (kKind == kMinimum) return min_propagate(acc, v);
  else if constexpr (kKind == kMaximum) return max_propagate(acc, v);
  else return acc + v;
}
// kMean divides once, at the very end; 0 / 0 gives the NaN of an empty mean.
template <int kKind> __device__ __forceinline__ float reduce_final(float acc, float divisor) {
  if constexpr (kKind == kMean) return acc / divisor;
  else return acc;
}

// ---- rows -------------------------------------------------------------------------------------
// kLanes lanes per (row, tile); unit = row * tiles + tile is also the output index.
template <class TIn, class TOut, int kKind, int kLanes, bool kVector>
__global__ __launch_bounds__(kBlockThreads) void reduce_rows(const void *x, void *y, uint32_t units,
                                                             uint32_t width, uint32_t tiles,
                                                             uint32_t tile_width, float divisor) {
  constexpr int kVec = Traits<TIn>::kVec;
  constexpr int kUnitsPerBlock = kBlockThreads / kLanes;
  __shared__ float joint[kBlockThreads / kWaveLanes];
  const uint32_t lane = threadIdx.x % kLanes;
  const uint32_t unit = blockIdx.x * kUnitsPerBlock + threadIdx.x / kLanes;
  const bool unit_ok = unit < units;
  float acc = reduce_identity<kKind>();
  if (unit_ok) {
    const uint32_t row = unit / tiles, tile = unit - row * tiles;
    const uint32_t begin = tile * tile_width;
    const uint32_t end = min(width, begin + tile_width);
    if constexpr (kVector) {
      // width and tile_width are multiples of the vector width
      const size_t base = (size_t)row * (width / kVec);
      const uint32_t last = end / kVec;
      uint32_t vec = begin / kVec + lane;
      for (; vec + 3 * kLanes < last; vec += 4 * kLanes) {
        u32x4 raw[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) raw[i] = load16_stream(x, base + vec + i * kLanes);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float v[kVec];
          Traits<TIn>::unpack(raw[i], v);
#pragma unroll
          for (int j = 0; j < kVec; ++j) acc = reduce_step<kKind>(acc, v[j]);
        }
      }
      for (; vec + kLanes < last; vec += 2 * kLanes) {
        u32x4 a = load16_stream(x, base + vec), b = load16_stream(x, base + vec + kLanes);
        float va[kVec], vb[kVec];
        Traits<TIn>::unpack(a, va);
        Traits<TIn>::unpack(b, vb);
#pragma unroll
        for (int j = 0; j < kVec; ++j) acc = reduce_step<kKind>(reduce_step<kKind>(acc, va[j]), vb[j]);
      }
      if (vec < last) {
        float v[kVec];
        Traits<TIn>::unpack(load16_stream(x, base + vec), v);
#pragma unroll
        for (int j = 0; j < kVec; ++j) acc = reduce_step<kKind>(acc, v[j]);
      }
    } else {
      const size_t base = (size_t)row * width;
      for (uint32_t i = begin + lane; i < end; i += kLanes)
        acc = reduce_step<kKind>(acc, Traits<TIn>::load(x, base + i));
    }
  }
  acc = row_reduce<kLanes>(acc, joint, [](float a, float b) { return reduce_step<kKind>(a, b); });
  if (unit_ok && lane == 0) Traits<TOut>::store(y, unit, reduce_final<kKind>(acc, divisor));
}

// ---- columns ----------------------------------------------------------------------------------
// Block of 256 threads = lanes_x along `inner` (units of one vector or one element) times
// lanes_y along `reduced`.  Grid: x = outer * x_tiles + tile of `inner`, y = segment of `reduced`.
// The output index of (segment, outer, column) is (segment * outer_count + outer) * inner +
// column: with one segment that is the final tensor, otherwise f32 partial results.
template <class TIn, class TOut, int kKind, bool kVector>
__global__ __launch_bounds__(kBlockThreads) void reduce_columns(const void *x, void *y,
                                                                uint32_t outer_count,
                                                                uint32_t reduced, uint32_t inner,
                                                                uint32_t lanes_x_log2, uint32_t x_tiles,
                                                                uint32_t segment_rows, float divisor) {
  constexpr int kW = kVector ? Traits<TIn>::kVec : 1;
  __shared__ float fold[kBlockThreads * kW];
  const uint32_t lanes_x = 1u << lanes_x_log2, lanes_y = kBlockThreads >> lanes_x_log2;
  const uint32_t tx = threadIdx.x & (lanes_x - 1), ty = threadIdx.x >> lanes_x_log2;
  const uint32_t units = inner / kW;
  const uint32_t outer = blockIdx.x / x_tiles, segment = blockIdx.y;
  const uint32_t unit = (blockIdx.x - outer * x_tiles) * lanes_x + tx;
  const bool active = unit < units;
  const uint32_t begin = segment * segment_rows;
  const uint32_t end = min(reduced, begin + segment_rows);

  float acc[kW];
#pragma unroll
  for (int j = 0; j < kW; ++j) acc[j] = reduce_identity<kKind>();
  if (active) {
    const size_t base = (size_t)outer * reduced * units + unit;  // in units
    uint32_t r = begin + ty;
    if constexpr (kVector) {
      for (; r + lanes_y < end; r += 2 * lanes_y) {
        u32x4 a = load16_stream(x, base + (size_t)r * units);
        u32x4 b = load16_stream(x, base + (size_t)(r + lanes_y) * units);
        float va[kW], vb[kW];
        Traits<TIn>::unpack(a, va);
        Traits<TIn>::unpack(b, vb);
#pragma unroll
        for (int j = 0; j < kW; ++j) acc[j] = reduce_step<kKind>(reduce_step<kKind>(acc[j], va[j]), vb[j]);
      }
      if (r < end) {
        float v[kW];
        Traits<TIn>::unpack(load16_stream(x, base + (size_t)r * units), v);
#pragma unroll
        for (int j = 0; j < kW; ++j) acc[j] = reduce_step<kKind>(acc[j], v[j]);
      }
    } else {
      for (; r < end; r += lanes_y)
        acc[0] = reduce_step<kKind>(acc[0], Traits<TIn>::load(x, base + (size_t)r * units));
    }
  }
  // fold the lanes_y partial results of a column (halving tree through LDS)
  for (uint32_t half = lanes_y >> 1; half > 0; half >>= 1) {
    if (ty >= half && ty < 2 * half) {
#pragma unroll
      for (int j = 0; j < kW; ++j) fold[threadIdx.x * kW + j] = acc[j];
    }
    __syncthreads();
    if (ty < half) {
      const uint32_t other = ((ty + half) << lanes_x_log2) + tx;
#pragma unroll
      for (int j = 0; j < kW; ++j) acc[j] = reduce_step<kKind>(acc[j], fold[other * kW + j]);
    }
    __syncthreads();
  }
  if (active && ty == 0) {
    const size_t out = ((size_t)segment * outer_count + outer) * inner + (size_t)unit * kW;
#pragma unroll
    for (int j = 0; j < kW; ++j) Traits<TOut>::store(y, out + j, reduce_final<kKind>(acc[j], divisor));
  }
}

// ---- general ----------------------------------------------------------------------------------
struct GeneralArgs {
  uint32_t rows, width;
  int32_t rank;
  uint32_t axes;
  uint32_t dims[kMaxRank];
  int64_t strides[kMaxRank];
};

template <class T> __device__ __forceinline__ float gather_bytes(const char *p) {
  uint32_t bits = 0;
#pragma unroll
  for (int b = 0; b < Traits<T>::kSize; ++b) bits |= (uint32_t)(uint8_t)p[b] << (8 * b);
  if constexpr (Traits<T>::kSize == 4) return bits_f32(bits);
  else {
    const uint16_t narrow = (uint16_t)bits;
    return Traits<T>::load(&narrow, 0);
  }
}

template <class T, int kKind, bool kBytewise>
__global__ __launch_bounds__(kBlockThreads) void reduce_general(const char *x, void *y, GeneralArgs g,
                                                                float divisor) {
  const uint32_t lane = threadIdx.x % kWaveLanes;
  const uint32_t row = blockIdx.x * (kBlockThreads / kWaveLanes) + threadIdx.x / kWaveLanes;
  const bool row_ok = row < g.rows;
  float acc = reduce_identity<kKind>();
  if (row_ok) {
    // the coordinates of the axes that are kept, once per result
    int64_t base = 0;
    uint32_t remaining = row;
    for (int axis = g.rank - 1; axis >= 0; --axis) {
      if ((g.axes >> axis) & 1u) continue;
      base += (int64_t)(remaining % g.dims[axis]) * g.strides[axis];
      remaining /= g.dims[axis];
    }
    for (uint32_t column = lane; column < g.width; column += kWaveLanes) {
      int64_t offset = base;
      remaining = column;
      for (int axis = g.rank - 1; axis >= 0; --axis) {
        if (!((g.axes >> axis) & 1u)) continue;
        offset += (int64_t)(remaining % g.dims[axis]) * g.strides[axis];
        remaining /= g.dims[axis];
      }
      const float v = kBytewise ? gather_bytes<T>(x + offset) : Traits<T>::load(x + offset, 0);
      acc = reduce_step<kKind>(acc, v);
    }
  }
  acc = group_reduce<kWaveLanes>(LaneF32{acc}, [](LaneF32 a, LaneF32 b) {
          return LaneF32{reduce_step<kKind>(a.x, b.x)};
        }).x;
  if (row_ok && lane == 0) Traits<T>::store(y, row, reduce_final<kKind>(acc, divisor));
}

// ---- host side --------------------------------------------------------------------------------
uint32_t ceil_div(uint64_t a, uint64_t b) { return (uint32_t)((a + b - 1) / b); }

// reduce_rows/<block|wave per unit>/<vector|scalar>, reduce_columns/<vector|scalar>, reduce_general[/bytes]
template <bool kBlock, bool kVector> struct RowsTag {
  static std::string text() { return std::string("reduce_rows/") + (kBlock ? "block" : "wave") + (kVector ? "/vector" : "/scalar"); }
};
template <bool kVector> struct ColumnsTag {
  static std::string text() { return std::string("reduce_columns/") + (kVector ? "vector" : "scalar"); }
};
template <bool kBytewise> struct GeneralTag {
  static std::string text() { return kBytewise ? "reduce_general/bytes" : "reduce_general"; }
};

template <class TIn, class TOut, int kKind>
void rows_launch(const void *x, void *y, uint32_t rows, uint32_t width, uint32_t tiles,
                 uint32_t tile_width, float divisor, bool vector, hipStream_t s) {
  const uint32_t units = rows * tiles;
  const bool wide = (size_t)std::min(width, tile_width) * Traits<TIn>::kSize >= 8192;
  if (wide && vector) note_variant<RowsTag<true, true>>();
  else if (wide) note_variant<RowsTag<true, false>>();
  else if (vector) note_variant<RowsTag<false, true>>();
  else note_variant<RowsTag<false, false>>();
  if (wide) {
    if (vector)
      hipLaunchKernelGGL((reduce_rows<TIn, TOut, kKind, kBlockThreads, true>), dim3(units),
                         dim3(kBlockThreads), 0, s, x, y, units, width, tiles, tile_width, divisor);
    else
      hipLaunchKernelGGL((reduce_rows<TIn, TOut, kKind, kBlockThreads, false>), dim3(units),
                         dim3(kBlockThreads), 0, s, x, y, units, width, tiles, tile_width, divisor);
  } else {
    const uint32_t blocks = ceil_div(units, kBlockThreads / kWaveLanes);
    if (vector)
      hipLaunchKernelGGL((reduce_rows<TIn, TOut, kKind, kWaveLanes, true>), dim3(blocks),
                         dim3(kBlockThreads), 0, s, x, y, units, width, tiles, tile_width, divisor);
    else
      hipLaunchKernelGGL((reduce_rows<TIn, TOut, kKind, kWaveLanes, false>), dim3(blocks),
                         dim3(kBlockThreads), 0, s, x, y, units, width, tiles, tile_width, divisor);
  }
}

// Lanes along `inner`: at most one wave (64 vectors = 1 KiB contiguous per row) and at least 8
// (128 B per row), the narrowest count that still yields about a thousand blocks: with few
// columns the blocks must come from cutting `inner` finely (measured on [8192, 2048] bf16 over
// axis 0: 19.8 us with 64 lanes along `inner`, 10.4-11.8 us with 8-32).
uint32_t lanes_x_log2_for(uint32_t units, uint32_t outer) {
  uint32_t log2 = 0;
  while (log2 < 6 && (1u << log2) < units) ++log2;
  while (log2 > 3 && (uint64_t)ceil_div(units, 1u << log2) * outer < 1024) --log2;
  return log2;
}

template <class TIn, class TOut, int kKind>
void columns_launch(const void *x, void *y, uint32_t outer, uint32_t reduced, uint32_t inner,
                    uint32_t segments, uint32_t segment_rows, float divisor, bool vector,
                    hipStream_t s) {
  const uint32_t units = vector ? inner / Traits<TIn>::kVec : inner;
  const uint32_t log2 = lanes_x_log2_for(units, outer);
  const uint32_t x_tiles = ceil_div(units, 1u << log2);
  const dim3 grid(x_tiles * outer, segments, 1);
  if (vector) note_variant<ColumnsTag<true>>();
  else note_variant<ColumnsTag<false>>();
  if (vector)
    hipLaunchKernelGGL((reduce_columns<TIn, TOut, kKind, true>), grid, dim3(kBlockThreads), 0, s, x, y,
                       outer, reduced, inner, log2, x_tiles, segment_rows, divisor);
  else
    hipLaunchKernelGGL((reduce_columns<TIn, TOut, kKind, false>), grid, dim3(kBlockThreads), 0, s, x, y,
                       outer, reduced, inner, log2, x_tiles, segment_rows, divisor);
}

template <class T, int kKind>
hipError_t run_kind(const ReduceParams &p, const void *x, void *y, void *workspace, bool in_vector,
                    hipStream_t s) {
  constexpr int kVec = Traits<T>::kVec;
  // the first of two dispatches never divides: a mean is a sum until the last step
  constexpr int kPartial = kKind == kMean ? kSum : kKind;
  switch (p.form) {
    case ReduceForm::kRows: {
      const bool vector = in_vector && p.width % kVec == 0;
      if (p.tiles <= 1) {
        rows_launch<T, T, kKind>(x, y, p.rows, p.width, 1, p.width, p.divisor, vector, s);
      } else {
        rows_launch<T, F32, kPartial>(x, workspace, p.rows, p.width, p.tiles, p.tile_width, 1.0f, vector, s);
        rows_launch<F32, T, kKind>(workspace, y, p.rows, p.tiles, 1, p.tiles, p.divisor, p.tiles % 4 == 0, s);
      }
      break;
    }
    case ReduceForm::kColumns: {
      const bool vector = in_vector && p.inner % kVec == 0;
      if (p.segments <= 1) {
        columns_launch<T, T, kKind>(x, y, p.outer, p.reduced, p.inner, 1, p.reduced, p.divisor, vector, s);
      } else {
        columns_launch<T, F32, kPartial>(x, workspace, p.outer, p.reduced, p.inner, p.segments,
                                         p.segment_rows, 1.0f, vector, s);
        const uint64_t flat = (uint64_t)p.outer * p.inner;  // the partial results: [segments, flat] f32
        columns_launch<F32, T, kKind>(workspace, y, 1, p.segments, (uint32_t)flat, 1, p.segments,
                                      p.divisor, flat % 4 == 0, s);
      }
      break;
    }
    case ReduceForm::kGeneral: {
      GeneralArgs g{};
      g.rows = p.rows;
      g.width = p.width;
      g.rank = p.rank;
      g.axes = p.axes;
      for (int a = 0; a < p.rank; ++a) {
        g.dims[a] = p.dims[a];
        g.strides[a] = p.strides[a];
      }
      const uint32_t blocks = ceil_div(p.rows, kBlockThreads / kWaveLanes);
      if (p.bytewise) note_variant<GeneralTag<true>>();
      else note_variant<GeneralTag<false>>();
      if (p.bytewise)
        hipLaunchKernelGGL((reduce_general<T, kKind, true>), dim3(blocks), dim3(kBlockThreads), 0, s,
                           static_cast<const char *>(x), y, g, p.divisor);
      else
        hipLaunchKernelGGL((reduce_general<T, kKind, false>), dim3(blocks), dim3(kBlockThreads), 0, s,
                           static_cast<const char *>(x), y, g, p.divisor);
      break;
    }
  }
  return hipGetLastError();
}

template <class T>
hipError_t run(const ReduceParams &p, const void *x, void *y, void *workspace, bool in_vector,
               hipStream_t s) {
  switch (p.kind) {
    case kSum: return run_kind<T, kSum>(p, x, y, workspace, in_vector, s);
    case kMean: return run_kind<T, kMean>(p, x, y, workspace, in_vector, s);
    case kMinimum: return run_kind<T, kMinimum>(p, x, y, workspace, in_vector, s);
    case kMaximum: return run_kind<T, kMaximum>(p, x, y, workspace, in_vector, s);
  }
  return hipErrorInvalidValue;
}

}  // namespace

// How a launch is cut: enough blocks to occupy every compute unit several times over, never
// pieces so small that the second dispatch dominates.
void reduce_plan(Elem type, ReduceParams *p) {
  const uint32_t size = type == Elem::kF32 ? 4 : 2;
  const uint32_t vec = 16 / size;
  p->tiles = 1;
  p->tile_width = p->width;
  p->segments = 1;
  p->segment_rows = p->reduced;
  p->workspace_bytes = 0;
  p->dispatches = 1;
  constexpr uint32_t kWantedBlocks = 2048;
  if (p->form == ReduceForm::kRows) {
    const uint64_t row_bytes = (uint64_t)p->width * size;
    if (p->rows < kWantedBlocks / 2 && row_bytes >= 128 * 1024) {
      // 32 KiB tiles: 16 to 256 KiB measured alike or worse on a 64 MiB row
      const uint32_t by_size = ceil_div(row_bytes, 32 * 1024);
      const uint32_t by_need = ceil_div(kWantedBlocks, p->rows);
      const uint32_t tiles = by_size < by_need ? by_size : by_need;
      const uint32_t quantum = vec * kBlockThreads * 2;  // whole double steps of a block
      p->tile_width = ceil_div(ceil_div(p->width, tiles), quantum) * quantum;
      p->tiles = ceil_div(p->width, p->tile_width);
      if (p->tiles > 1) {
        p->workspace_bytes = (size_t)p->rows * p->tiles * sizeof(float);
        p->dispatches = 2;
      } else {
        p->tile_width = p->width;
      }
    }
  } else if (p->form == ReduceForm::kColumns) {
    const uint32_t units = p->inner % vec == 0 ? p->inner / vec : p->inner;
    const uint32_t log2 = lanes_x_log2_for(units, p->outer);
    const uint32_t lanes_y = kBlockThreads >> log2;
    const uint64_t blocks = (uint64_t)ceil_div(units, 1u << log2) * p->outer;
    const uint32_t rows_per_step = lanes_y * 8;  // a segment keeps every lane busy for >= 8 rows
    const uint64_t input_bytes = (uint64_t)p->outer * p->reduced * p->inner * size;
    if (blocks < kWantedBlocks / 2 && p->reduced >= 2 * rows_per_step && input_bytes >= 512 * 1024) {
      const uint32_t by_need = ceil_div(kWantedBlocks, blocks);
      uint32_t by_size = p->reduced / rows_per_step;
      // the partial results are written and read again: keep them under 1/64 of the elements
      if (by_size > p->reduced / 64) by_size = p->reduced / 64;
      if (by_size == 0) by_size = 1;
      uint32_t segments = by_need < by_size ? by_need : by_size;
      if (segments > 65535) segments = 65535;
      p->segment_rows = ceil_div(p->reduced, segments);
      p->segments = ceil_div(p->reduced, p->segment_rows);
      if (p->segments > 1) {
        p->workspace_bytes = (size_t)p->segments * p->outer * p->inner * sizeof(float);
        p->dispatches = 2;
      } else {
        p->segment_rows = p->reduced;
      }
    }
  }
}

hipError_t launch_reduce(Elem type, const ReduceParams &p, const void *x, void *y, void *workspace,
                         bool input_vector_aligned, hipStream_t stream) {
  if (p.rows == 0) return hipSuccess;
  switch (type) {
    case Elem::kF32: return run<F32>(p, x, y, workspace, input_vector_aligned, stream);
    case Elem::kF16: return run<F16>(p, x, y, workspace, input_vector_aligned, stream);
    case Elem::kBF16: return run<BF16>(p, x, y, workspace, input_vector_aligned, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace hyle_hip
