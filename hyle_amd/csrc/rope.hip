// RoPE with explicit frequencies (include/hyle/compute/operation.h:388-392; schema
// src/compute_ops/operation.cc:639-696,1566-1574).  The arithmetic is the reference's ggml route's
// (src/compute_ggml_runtime/explicit_rope.h:11-74): everything in f32, phase = frequency * position
// with the position converted to f32 first, cos and sin of the phase, and for a pair (a, b)
//   a' = a * cos - b * sin,   b' = a * sin + b * cos
// every product and sum rounded on its own; narrow storage is widened on load and rounded once on
// store; elements past rotary_dimensions pass through bit for bit.  Pairs are neighbours
// (2i, 2i + 1) in the interleaved layout and (i, i + rotary / 2) in the half-split one.
#include "device_common.h"
#include "kernels.h"

namespace hyle_hip {
namespace {

struct RopeOperands {
  const void *positions;
  const float *frequencies;
  uint32_t depth, rotary, pairs, sequence, inner;
  bool wide_positions, batched_positions, stepped_frequencies;
};

// The f32 position of a row and where its frequencies start.
__device__ __forceinline__ float row_position(const RopeOperands &p, uint32_t row, uint32_t *frequency_first) {
  const uint32_t step_index = row / p.inner, step = step_index % p.sequence;
  const uint32_t at = p.batched_positions ? step_index : step;  // [prefix..., S] flattens to step_index
  *frequency_first = p.stepped_frequencies ? step * p.pairs : 0u;
  return p.wide_positions ? (float)static_cast<const int64_t *>(p.positions)[at]
                          : (float)static_cast<const int32_t *>(p.positions)[at];
}

__device__ __forceinline__ void rotate(float a, float b, float phase, float *first, float *second) {
  float s, c;
  sincosf(phase, &s, &c);
  *first = a * c - b * s;
  *second = a * s + b * c;
}

// For rotary widths whose table of phases would not fit LDS.  Rows that share a sequence step (the
// heads of a token) share their phases: a thread owns one
// vector place of the row -- in the half-split layout a first-half vector and its partner in the
// second half -- takes cos and sin of its pairs once and applies them to up to kRowsPerThread
// consecutive rows of the step.  Places past the rotary width copy the tail.
constexpr uint32_t kRowsPerThread = 8;
template <class T, bool kHalfSplit>
__global__ __launch_bounds__(kBlockThreads) void rope_vectors(RopeOperands p, const void *in, void *out, uint32_t vectors_per_row,
                                                              uint32_t places, uint32_t groups, uint32_t units) {
  constexpr int kVec = Traits<T>::kVec;
  constexpr int kPairs = kHalfSplit ? kVec : kVec / 2;  // pairs a thread rotates per row
  const uint32_t g = blockIdx.x * kBlockThreads + threadIdx.x;
  if (g >= units) return;
  const uint32_t place = g % places, rest = g / places;
  const uint32_t group = rest % groups, step_index = rest / groups;
  const uint32_t rotating = (kHalfSplit ? p.pairs : p.rotary) / kVec;  // places that rotate; the others copy the tail
  const uint32_t first_row = group * kRowsPerThread;
  const uint32_t last_row = first_row + kRowsPerThread < p.inner ? first_row + kRowsPerThread : p.inner;
  const size_t base = ((size_t)step_index * p.inner) * vectors_per_row;
  if (place >= rotating) {
    const uint32_t v = p.rotary / kVec + (place - rotating);
    for (uint32_t h = first_row; h < last_row; ++h) {
      const size_t at = base + (size_t)h * vectors_per_row + v;
      store16_stream(out, at, load16_stream(in, at));
    }
    return;
  }
  const uint32_t step = step_index % p.sequence;
  const uint32_t position_at = p.batched_positions ? step_index : step;  // [prefix..., S] flattens to step_index
  const float position = p.wide_positions ? (float)static_cast<const int64_t *>(p.positions)[position_at]
                                          : (float)static_cast<const int32_t *>(p.positions)[position_at];
  const float *frequencies = p.frequencies + (p.stepped_frequencies ? step * p.pairs : 0u) + place * kPairs;
  float c[kPairs], s[kPairs];
#pragma unroll
  for (int j = 0; j < kPairs; ++j) sincosf(frequencies[j] * position, &s[j], &c[j]);
  const uint32_t partner = p.pairs / kVec;  // vectors between the halves of a pair (half-split)
  constexpr uint32_t kBatch = 4;  // rows whose loads are in flight together
  for (uint32_t h0 = first_row; h0 < last_row; h0 += kBatch) {
    u32x4 lower[kBatch], upper[kBatch];
    size_t at[kBatch];
#pragma unroll
    for (uint32_t k = 0; k < kBatch; ++k) {
      const uint32_t h = h0 + k < last_row ? h0 + k : last_row - 1;  // a row past the end reads the last one again
      at[k] = base + (size_t)h * vectors_per_row + place;
      lower[k] = load16_stream(in, at[k]);
      if constexpr (kHalfSplit) upper[k] = load16_stream(in, at[k] + partner);
    }
#pragma unroll
    for (uint32_t k = 0; k < kBatch; ++k) {
      if (h0 + k >= last_row) break;
      if constexpr (kHalfSplit) {
        float a[kVec], b[kVec], ra[kVec], rb[kVec];
        Traits<T>::unpack(lower[k], a);
        Traits<T>::unpack(upper[k], b);
#pragma unroll
        for (int j = 0; j < kVec; ++j) {
          ra[j] = a[j] * c[j] - b[j] * s[j];
          rb[j] = a[j] * s[j] + b[j] * c[j];
        }
        store16_stream(out, at[k], Traits<T>::pack(ra));
        store16_stream(out, at[k] + partner, Traits<T>::pack(rb));
      } else {
        float x[kVec], r[kVec];
        Traits<T>::unpack(lower[k], x);
#pragma unroll
        for (int j = 0; j < kVec / 2; ++j) {
          r[2 * j] = x[2 * j] * c[j] - x[2 * j + 1] * s[j];
          r[2 * j + 1] = x[2 * j] * s[j] + x[2 * j + 1] * c[j];
        }
        store16_stream(out, at[k], Traits<T>::pack(r));
      }
    }
  }
}

// The same with the phases of a step taken once for all its rows: a block owns `steps_per_block`
// consecutive sequence steps (all `inner` rows of each, contiguous in memory), leaves cos and sin
// of their pairs in LDS and then walks the steps' vector places, a thread per place and row.
template <class T, bool kHalfSplit>
__global__ __launch_bounds__(kBlockThreads) void rope_steps(RopeOperands p, const void *in, void *out, uint32_t vectors_per_row,
                                                            uint32_t places, uint32_t steps_per_block, uint32_t steps) {
  extern __shared__ float table[];  // per step of the block: cos of the pairs, then sin
  constexpr int kVec = Traits<T>::kVec;
  constexpr int kPairs = kHalfSplit ? kVec : kVec / 2;
  const uint32_t first_step = blockIdx.x * steps_per_block;
  const uint32_t own = steps - first_step < steps_per_block ? steps - first_step : steps_per_block;
  for (uint32_t i = threadIdx.x; i < own * p.pairs; i += kBlockThreads) {
    const uint32_t local = i / p.pairs, pair = i - local * p.pairs;
    const uint32_t step_index = first_step + local, step = step_index % p.sequence;
    const uint32_t position_at = p.batched_positions ? step_index : step;
    const float position = p.wide_positions ? (float)static_cast<const int64_t *>(p.positions)[position_at]
                                            : (float)static_cast<const int32_t *>(p.positions)[position_at];
    const float frequency = p.frequencies[(p.stepped_frequencies ? step * p.pairs : 0u) + pair];
    sincosf(frequency * position, &table[(2 * local + 1) * p.pairs + pair], &table[2 * local * p.pairs + pair]);
  }
  __syncthreads();
  const uint32_t rotating = (kHalfSplit ? p.pairs : p.rotary) / kVec, partner = p.pairs / kVec;
  const uint32_t per_step = p.inner * places, total = own * per_step;
  // a unit is one place of one row; its loads are issued one unit ahead of its arithmetic
  struct Unit {
    size_t at;        // the vector in the tensor
    uint32_t table;   // where the unit's cos values start; 0xFFFFFFFF: a tail vector that is copied
    u32x4 lower, upper;
  };
  auto fetch = [&](uint32_t u) {
    Unit unit;
    const uint32_t local = u / per_step, within = u - local * per_step;
    const uint32_t h = within / places, place = within - h * places;
    const size_t row = ((size_t)(first_step + local) * p.inner + h) * vectors_per_row;
    if (place >= rotating) {
      unit.at = row + p.rotary / kVec + (place - rotating);
      unit.table = 0xFFFFFFFFu;
      unit.lower = load16_stream(in, unit.at);
      unit.upper = unit.lower;
    } else {
      unit.at = row + place;
      unit.table = 2 * local * p.pairs + place * kPairs;
      unit.lower = load16_stream(in, unit.at);
      unit.upper = kHalfSplit ? load16_stream(in, unit.at + partner) : unit.lower;
    }
    return unit;
  };
  uint32_t u = threadIdx.x;
  if (u >= total) return;
  Unit current = fetch(u);
  while (true) {
    const uint32_t following = u + kBlockThreads;
    Unit next = current;
    if (following < total) next = fetch(following);
    if (current.table == 0xFFFFFFFFu) {
      store16_stream(out, current.at, current.lower);
    } else {
      const float *c = table + current.table, *s = c + p.pairs;
      if constexpr (kHalfSplit) {
        float a[kVec], b[kVec], ra[kVec], rb[kVec];
        Traits<T>::unpack(current.lower, a);
        Traits<T>::unpack(current.upper, b);
#pragma unroll
        for (int j = 0; j < kVec; ++j) {
          ra[j] = a[j] * c[j] - b[j] * s[j];
          rb[j] = a[j] * s[j] + b[j] * c[j];
        }
        store16_stream(out, current.at, Traits<T>::pack(ra));
        store16_stream(out, current.at + partner, Traits<T>::pack(rb));
      } else {
        float x[kVec], r[kVec];
        Traits<T>::unpack(current.lower, x);
#pragma unroll
        for (int j = 0; j < kVec / 2; ++j) {
          r[2 * j] = x[2 * j] * c[j] - x[2 * j + 1] * s[j];
          r[2 * j + 1] = x[2 * j] * s[j] + x[2 * j + 1] * c[j];
        }
        store16_stream(out, current.at, Traits<T>::pack(r));
      }
    }
    if (following >= total) break;
    current = next;
    u = following;
  }
}

// Any depth, rotary width and alignment: a thread per pair, then per tail element.
template <class T>
__global__ __launch_bounds__(kBlockThreads) void rope_elements(RopeOperands p, const void *in, void *out, bool half_split,
                                                               uint32_t units_per_row, uint64_t units) {
  const uint64_t g = (uint64_t)blockIdx.x * kBlockThreads + threadIdx.x;
  if (g >= units) return;
  const uint32_t row = (uint32_t)(g / units_per_row), unit = (uint32_t)(g - (uint64_t)row * units_per_row);
  const size_t base = (size_t)row * p.depth;
  if (unit >= p.pairs) {
    const size_t at = base + p.rotary + (unit - p.pairs);
    if constexpr (Traits<T>::kSize == 4) static_cast<uint32_t *>(out)[at] = static_cast<const uint32_t *>(in)[at];
    else static_cast<uint16_t *>(out)[at] = static_cast<const uint16_t *>(in)[at];
    return;
  }
  uint32_t frequency_first;
  const float position = row_position(p, row, &frequency_first);
  const size_t first = base + (half_split ? unit : 2 * unit), second = half_split ? first + p.pairs : first + 1;
  float a, b;
  rotate(Traits<T>::load(in, first), Traits<T>::load(in, second), p.frequencies[frequency_first + unit] * position, &a, &b);
  Traits<T>::store(out, first, a);
  Traits<T>::store(out, second, b);
}

// Launch-shape labels
template <int kForm, bool kHalfSplit> struct RopeTag {  // 0 steps, 1 vectors
  static std::string text() { return std::string(kForm == 0 ? "rope_steps/" : "rope_vectors/") + (kHalfSplit ? "half-split" : "interleaved"); }
};
struct RopeElementsTag {
  static std::string text() { return "rope_elements"; }
};

template <class T>
hipError_t run_rope(const RopeParams &p, const void *in, const void *positions, const void *frequencies, void *out,
                    bool vector_aligned, hipStream_t stream) {
  constexpr uint32_t kVec = Traits<T>::kVec;
  const RopeOperands o{positions, static_cast<const float *>(frequencies), p.depth, p.rotary, p.rotary / 2, p.sequence, p.inner,
                       p.wide_positions, p.batched_positions, p.stepped_frequencies};
  const bool whole = p.depth % kVec == 0 && p.rotary % kVec == 0 && (!p.half_split || (p.rotary / 2) % kVec == 0);
  const dim3 block(kBlockThreads);
  if (vector_aligned && whole) {
    const uint32_t per_row = p.depth / kVec;
    const uint32_t places = (p.half_split ? p.rotary / 2 : p.rotary) / kVec + (p.depth - p.rotary) / kVec;
    const uint32_t groups = (p.inner + kRowsPerThread - 1) / kRowsPerThread;
    const uint64_t units = p.rows / p.inner * groups * places;  // at most INT32_MAX elements / kVec
    const uint64_t steps = p.rows / p.inner;
    if (p.rotary / 2 <= 2048) {
      // The steps that give a block about 512 places, two per thread with the second one's loads
      // issued before the first one's arithmetic.  Measured on MI355X for [1, 8192, 16, 128] bf16,
      // half-split: 13.5 us so (14.2 / 13.6 / 13.8 / 15.3 us with 128 / 256 / 1024 / 2048 places);
      // 14.9 us when every thread takes cos and sin itself for eight rows, 31.2 us when it does
      // so for each row; the plain copy of the same bytes 11.1 us.
      uint32_t per_block = 512 / (p.inner * places);
      per_block = per_block < 1 ? 1 : per_block;
      while (per_block > 1 && (size_t)per_block * p.rotary * sizeof(float) > 32768) --per_block;
      const size_t lds = (size_t)per_block * p.rotary * sizeof(float);
      const dim3 grid((uint32_t)((steps + per_block - 1) / per_block));
      if (p.half_split) {
        note_variant<RopeTag<0, true>>();
        hipLaunchKernelGGL((rope_steps<T, true>), grid, block, lds, stream, o, in, out, per_row, places, per_block, (uint32_t)steps);
      } else {
        note_variant<RopeTag<0, false>>();
        hipLaunchKernelGGL((rope_steps<T, false>), grid, block, lds, stream, o, in, out, per_row, places, per_block, (uint32_t)steps);
      }
      return hipGetLastError();
    }
    const dim3 grid((uint32_t)((units + kBlockThreads - 1) / kBlockThreads));
    if (p.half_split) {
      note_variant<RopeTag<1, true>>();
      hipLaunchKernelGGL((rope_vectors<T, true>), grid, block, 0, stream, o, in, out, per_row, places, groups, (uint32_t)units);
    } else {
      note_variant<RopeTag<1, false>>();
      hipLaunchKernelGGL((rope_vectors<T, false>), grid, block, 0, stream, o, in, out, per_row, places, groups, (uint32_t)units);
    }
    return hipGetLastError();
  }
  const uint32_t per_row = p.rotary / 2 + (p.depth - p.rotary);
  const uint64_t units = p.rows * per_row;
  note_variant<RopeElementsTag>();
  hipLaunchKernelGGL((rope_elements<T>), dim3((uint32_t)((units + kBlockThreads - 1) / kBlockThreads)), block, 0, stream, o, in,
                     out, p.half_split, per_row, units);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_rope(Elem type, const RopeParams &p, const void *in, const void *positions, const void *frequencies, void *out,
                       bool vector_aligned, hipStream_t stream) {
  if (p.rows == 0 || p.depth == 0) return hipSuccess;
  switch (type) {
    case Elem::kF32: return run_rope<F32>(p, in, positions, frequencies, out, vector_aligned, stream);
    case Elem::kF16: return run_rope<F16>(p, in, positions, frequencies, out, vector_aligned, stream);
    case Elem::kBF16: return run_rope<BF16>(p, in, positions, frequencies, out, vector_aligned, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace hyle_hip
