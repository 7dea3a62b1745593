// TopK(count = k) along one axis: values and int32 indices of the k best elements of every row,
// best first.
//
// Ordering is the reference's (tests/compute_route_vulkan/topk_test_support.h:62-76, the
// independent host ordering its device tests are held to; src/compute_provider_cuda/
// collectives.cu:405-421 builds the same order as a 64-bit key): numbers come before NaNs,
// larger first (smaller first when `largest` is off), equal numbers -- -0 and +0 are equal --
// and NaNs keep their index order.  Values are copies of the source bits
// (include/hyle/compute/providers/cuda.h:113-116).
//
// Every element becomes a unique 64-bit key, (ordered value << 32) | ~index, so that "best
// first" is plain descending integer order and no comparison ever ties.  A block sorts a tile of
// 2048 keys in LDS (bitonic network) and keeps its first k; lists of k keys are then merged
// 2048 / k at a time by the same sort until one list per row is left, which the last dispatch
// turns into the two outputs.  The lists live in the caller's workspace.
//
// Sorting whole tiles is bound by LDS traffic (66 passes over 16 KiB per tile).  For k <= 256 a
// block therefore *selects* instead: every thread keeps its share of the keys in registers, the
// k-th largest of the 256 per-thread maxima is a lower bound of the tile's k-th largest key
// (at least k keys reach it), and only the keys that reach that bound -- for unordered data a
// little more than k -- go to LDS to be sorted.  When more than 2048 keys reach it (ordered
// data can do that) the exact k-th key is found bit by bit with block-wide counts instead.
#include <algorithm>
#include <type_traits>

#include "device_common.h"
#include "kernels.h"

namespace hyle_hip {
namespace {

constexpr uint32_t kTile = 2048;  // keys one block sorts: 16 KiB of LDS

struct Addressing {
  uint32_t width, inner, count;  // extent of the axis, elements after it, k
  uint32_t dense_last;           // 1: dense tensor, axis innermost
  int32_t rank, axis;
  uint32_t dims[kMaxRank];
  int64_t strides[kMaxRank];
};

// Byte offset of element 0 of `row` (row = outer * inner + position after the axis).
__device__ __forceinline__ int64_t row_base(const Addressing &a, uint32_t row, uint32_t size) {
  if (a.dense_last) return (int64_t)row * a.width * size;
  int64_t base = 0;
  uint32_t remaining = row;
  for (int axis = a.rank - 1; axis >= 0; --axis) {
    if (axis == a.axis) continue;
    base += (int64_t)(remaining % a.dims[axis]) * a.strides[axis];
    remaining /= a.dims[axis];
  }
  return base;
}

// Element types: the three float storage types and int32 (include/hyle/compute/providers/cuda.h:108-121).
struct I32 {};
template <class T> struct KeyTraits {
  static constexpr int kSize = Traits<T>::kSize;
  static constexpr int kVec = Traits<T>::kVec;
};
template <> struct KeyTraits<I32> {
  static constexpr int kSize = 4;
  static constexpr int kVec = 4;
};

template <class T, bool kBytewise>
__device__ __forceinline__ uint32_t load_bits(const char *p) {
  constexpr int kSize = KeyTraits<T>::kSize;
  if constexpr (kBytewise) {
    uint32_t bits = 0;
#pragma unroll
    for (int b = 0; b < kSize; ++b) bits |= (uint32_t)(uint8_t)p[b] << (8 * b);
    return bits;
  } else if constexpr (kSize == 4) {
    return *reinterpret_cast<const uint32_t *>(p);
  } else {
    return *reinterpret_cast<const uint16_t *>(p);
  }
}
template <class T> __device__ __forceinline__ float bits_value(uint32_t bits) {
  if constexpr (KeyTraits<T>::kSize == 4) return bits_f32(bits);
  else {
    const uint16_t narrow = (uint16_t)bits;
    return Traits<T>::load(&narrow, 0);
  }
}

// The ordered half of a key from an element's storage bits: larger = better.  A NaN is 0 and
// sits below every number; -0 and +0 are one value.  int32 orders as a signed integer.
__device__ __forceinline__ uint32_t ordered_value(float v, bool largest) {
  if (v != v) return 0;
  const uint32_t bits = v == 0.0f ? 0u : f32_bits(v);
  const uint32_t ordered = bits ^ ((uint32_t)((int32_t)bits >> 31) | 0x80000000u);
  return largest ? ordered : ~ordered;
}
template <class T> __device__ __forceinline__ uint32_t ordered_bits(uint32_t bits, bool largest) {
  if constexpr (std::is_same<T, I32>::value) {
    const uint32_t ordered = bits ^ 0x80000000u;
    return largest ? ordered : ~ordered;
  } else {
    return ordered_value(bits_value<T>(bits), largest);
  }
}
// The storage bits of the kVec elements of a 16-byte vector.
template <class T> __device__ __forceinline__ void vector_bits(u32x4 raw, uint32_t (&bits)[KeyTraits<T>::kVec]) {
  const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
  if constexpr (KeyTraits<T>::kSize == 4) {
#pragma unroll
    for (int j = 0; j < 4; ++j) bits[j] = words[j];
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) bits[j] = (words[j / 2] >> (16 * (j % 2))) & 0xFFFFu;
  }
}
// A whole key: 0 is no element.
template <class T> __device__ __forceinline__ uint64_t make_key(uint32_t bits, uint32_t index, bool largest) {
  return ((uint64_t)ordered_bits<T>(bits, largest) << 32) | (uint32_t)~index;
}

// Descending bitonic sort of keys[0 .. n), n a power of two <= kTile; every thread of the block.
__device__ __forceinline__ void sort_descending(uint64_t *keys, uint32_t n) {
  for (uint32_t size = 2; size <= n; size <<= 1) {
    for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
      __syncthreads();
      for (uint32_t pair = threadIdx.x; pair < n / 2; pair += kBlockThreads) {
        const uint32_t lo = 2 * pair - (pair & (stride - 1));
        const uint32_t hi = lo + stride;
        const bool descending = (lo & size) == 0;
        const uint64_t a = keys[lo], b = keys[hi];
        if ((a < b) == descending) {
          keys[lo] = b;
          keys[hi] = a;
        }
      }
    }
  }
  __syncthreads();
}

// The first `count` keys of a sorted list -> outputs (kFinal) or the next list in the workspace.
template <class T, bool kBytewise, bool kFinal>
__device__ __forceinline__ void emit(const uint64_t *keys, const Addressing &a, uint32_t row,
                                     const char *x, void *values, int32_t *indices, uint64_t *list) {
  constexpr int kSize = KeyTraits<T>::kSize;
  if constexpr (kFinal) {
    const int64_t base = row_base(a, row, kSize);
    const int64_t step = a.dense_last ? kSize : a.strides[a.axis];
    const uint32_t outer = row / a.inner, position = row - outer * a.inner;
    for (uint32_t j = threadIdx.x; j < a.count; j += kBlockThreads) {
      // a list always holds `count` elements of the row here; the clamp only keeps a corrupted
      // workspace from turning into a wild address
      const uint32_t index = min(~(uint32_t)keys[j], a.width - 1);
      const uint32_t bits = load_bits<T, kBytewise>(x + base + (int64_t)index * step);
      const size_t out = ((size_t)outer * a.count + j) * a.inner + position;
      if constexpr (kSize == 4) static_cast<uint32_t *>(values)[out] = bits;
      else static_cast<uint16_t *>(values)[out] = (uint16_t)bits;
      indices[out] = (int32_t)index;
    }
  } else {
    for (uint32_t j = threadIdx.x; j < a.count; j += kBlockThreads) list[j] = keys[j];
  }
}

// One block per (row, tile): keys of up to kTile elements, sorted, best `count` kept.
template <class T, bool kVector, bool kBytewise, bool kFinal>
__global__ __launch_bounds__(kBlockThreads) void topk_tiles(const char *x, void *values, int32_t *indices,
                                                            uint64_t *lists, Addressing a, uint32_t tiles,
                                                            uint32_t sort_n, uint32_t largest) {
  constexpr int kSize = KeyTraits<T>::kSize;
  constexpr int kVec = KeyTraits<T>::kVec;
  __shared__ uint64_t keys[kTile];
  const uint32_t row = blockIdx.x / tiles, tile = blockIdx.x - row * tiles;
  const uint32_t first = tile * kTile;
  const int64_t base = row_base(a, row, kSize);
  if constexpr (kVector) {
    // dense rows whose starts are 16-byte aligned: whole vectors, a ragged end cannot occur
    const u32x4 *vectors = reinterpret_cast<const u32x4 *>(x + base);
    for (uint32_t v = threadIdx.x; v < sort_n / kVec; v += kBlockThreads) {
      const uint32_t element = first + v * kVec;
      if (element < a.width) {
        uint32_t bits[kVec];
        vector_bits<T>(__builtin_nontemporal_load(vectors + element / kVec), bits);
#pragma unroll
        for (int j = 0; j < kVec; ++j) keys[v * kVec + j] = make_key<T>(bits[j], element + j, largest != 0);
      } else {
#pragma unroll
        for (int j = 0; j < kVec; ++j) keys[v * kVec + j] = 0;
      }
    }
  } else {
    const int64_t step = a.dense_last ? kSize : a.strides[a.axis];
    for (uint32_t i = threadIdx.x; i < sort_n; i += kBlockThreads) {
      const uint32_t element = first + i;
      keys[i] = element < a.width
                    ? make_key<T>(load_bits<T, kBytewise>(x + base + (int64_t)element * step), element, largest != 0)
                    : 0;
    }
  }
  sort_descending(keys, sort_n);
  emit<T, kBytewise, kFinal>(keys, a, row, x, values, indices,
                             lists + ((size_t)row * tiles + tile) * a.count);
}

// One block per (row, group of `fan` lists): merge by sorting, keep the best `count`.
template <class T, bool kBytewise, bool kFinal>
__global__ __launch_bounds__(kBlockThreads) void topk_merge(const char *x, void *values, int32_t *indices,
                                                            const uint64_t *in_lists, uint64_t *out_lists,
                                                            Addressing a, uint32_t lists_in, uint32_t fan,
                                                            uint32_t lists_out, uint32_t sort_n) {
  __shared__ uint64_t keys[kTile];
  const uint32_t row = blockIdx.x / lists_out, group = blockIdx.x - row * lists_out;
  const uint32_t first_list = group * fan;
  const uint32_t taken = min(fan, lists_in - first_list) * a.count;
  const uint64_t *source = in_lists + ((size_t)row * lists_in + first_list) * a.count;
  for (uint32_t i = threadIdx.x; i < sort_n; i += kBlockThreads) keys[i] = i < taken ? source[i] : 0;
  sort_descending(keys, sort_n);
  emit<T, kBytewise, kFinal>(keys, a, row, x, values, indices,
                             out_lists + ((size_t)row * lists_out + group) * a.count);
}

// ---- counts above kTile / 2: whole sorted tiles, merged two runs at a time -------------------
// A run is a descending list of keys padded with zeros (no element) to a whole number of tiles.
// One block writes kTile keys of the merged run: a binary search along its diagonal (merge path)
// finds how many of the keys before its window come from each input run; the two windows, the
// second one reversed, form a bitonic sequence of 2 * kTile keys that one bitonic merge puts in
// order; its first half is the block's output.
__global__ __launch_bounds__(kBlockThreads) void topk_merge_runs(const uint64_t *in, uint64_t *out, uint32_t runs_in,
                                                                uint32_t run_in_keys, uint32_t runs_out,
                                                                uint32_t run_out_keys) {
  __shared__ uint64_t keys[2 * kTile];
  __shared__ uint32_t split;
  const uint32_t chunks = run_out_keys / kTile;
  const uint32_t chunk = blockIdx.x % chunks, run = (blockIdx.x / chunks) % runs_out, row = blockIdx.x / (chunks * runs_out);
  const uint64_t *a = in + ((size_t)row * runs_in + 2 * run) * run_in_keys;
  const bool paired = 2 * run + 1 < runs_in;
  const uint64_t *b = a + run_in_keys;  // read only when paired
  const uint32_t length_a = run_in_keys, length_b = paired ? run_in_keys : 0;
  const uint32_t diagonal = chunk * kTile;
  if (threadIdx.x == 0) {
    uint32_t low = diagonal > length_b ? diagonal - length_b : 0, high = diagonal < length_a ? diagonal : length_a;
    while (low < high) {
      const uint32_t mid = (low + high) / 2;  // mid keys of a and diagonal - mid of b before the window?
      if (a[mid] > b[diagonal - mid - 1]) low = mid + 1;  // a[mid] outranks the last key taken from b: take more of a
      else high = mid;
    }
    split = low;
  }
  __syncthreads();
  const uint32_t from_a = split, from_b = diagonal - split;
  for (uint32_t i = threadIdx.x; i < kTile; i += kBlockThreads) {
    keys[i] = from_a + i < length_a ? a[from_a + i] : 0;
    keys[2 * kTile - 1 - i] = from_b + i < length_b ? b[from_b + i] : 0;
  }
  for (uint32_t stride = kTile; stride > 0; stride >>= 1) {
    __syncthreads();
    for (uint32_t pair = threadIdx.x; pair < kTile; pair += kBlockThreads) {
      const uint32_t lo = 2 * pair - (pair & (stride - 1)), hi = lo + stride;
      const uint64_t first = keys[lo], second = keys[hi];
      if (first < second) {
        keys[lo] = second;
        keys[hi] = first;
      }
    }
  }
  __syncthreads();
  uint64_t *target = out + ((size_t)row * runs_out + run) * run_out_keys + diagonal;
  for (uint32_t i = threadIdx.x; i < kTile; i += kBlockThreads) target[i] = keys[i];
}

// The first `count` keys of every row's single run -> the two outputs.
template <class T, bool kBytewise>
__global__ __launch_bounds__(kBlockThreads) void topk_emit_run(const char *x, void *values, int32_t *indices,
                                                              const uint64_t *runs, Addressing a, uint32_t run_keys,
                                                              uint32_t blocks_per_row) {
  constexpr int kSize = KeyTraits<T>::kSize;
  const uint32_t row = blockIdx.x / blocks_per_row;
  const uint32_t j = (blockIdx.x % blocks_per_row) * kBlockThreads + threadIdx.x;
  if (j >= a.count) return;
  const int64_t base = row_base(a, row, kSize);
  const int64_t step = a.dense_last ? kSize : a.strides[a.axis];
  const uint32_t outer = row / a.inner, position = row - outer * a.inner;
  const uint32_t index = min(~(uint32_t)runs[(size_t)row * run_keys + j], a.width - 1);
  const uint32_t bits = load_bits<T, kBytewise>(x + base + (int64_t)index * step);
  const size_t at = ((size_t)outer * a.count + j) * a.inner + position;
  if constexpr (kSize == 4) static_cast<uint32_t *>(values)[at] = bits;
  else static_cast<uint16_t *>(values)[at] = (uint16_t)bits;
  indices[at] = (int32_t)index;
}

constexpr uint32_t kSelectMax = kBlockThreads;  // largest count the select route serves

// Exclusive prefix sum of `v` over the block in thread order; *total = sum over the block.
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t v, uint32_t *wave_totals, uint32_t *total) {
  const uint32_t lane = threadIdx.x % kWaveLanes, wave = threadIdx.x / kWaveLanes;
  uint32_t inclusive = v;
#pragma unroll
  for (int d = 1; d < kWaveLanes; d <<= 1) {
    const uint32_t other = __shfl_up(inclusive, d, kWaveLanes);
    if (lane >= (uint32_t)d) inclusive += other;
  }
  if (lane == kWaveLanes - 1) wave_totals[wave] = inclusive;
  __syncthreads();
  uint32_t before = 0, all = 0;
#pragma unroll
  for (uint32_t w = 0; w < kBlockThreads / kWaveLanes; ++w) {
    const uint32_t t = wave_totals[w];
    if (w < wave) before += t;
    all += t;
  }
  __syncthreads();
  *total = all;
  return before + inclusive - v;
}

// One block per (row, unit).  kFromLists = false: unit = a tile of 256 * kE elements of the row.
// kFromLists = true: unit = a group of `fan` lists of `count` keys left by an earlier dispatch.
// A thread keeps its kE keys as two words, hi (ordered value) and lo (~index; the compiler
// recomputes it from the slot number for elements); an empty slot is hi = lo = 0.
template <class T, int kE, bool kFromLists, bool kVector, bool kBytewise, bool kFinal>
__global__ __launch_bounds__(kBlockThreads) void topk_select(const char *x, void *values, int32_t *indices,
                                                             const uint64_t *in_lists, uint64_t *out_lists,
                                                             Addressing a, uint32_t units_in, uint32_t fan,
                                                             uint32_t units_out, uint32_t largest) {
  constexpr int kSize = KeyTraits<T>::kSize;
  constexpr int kVec = KeyTraits<T>::kVec;
  __shared__ uint64_t keys[kTile];  // kBlockThreads < kTile / 2: keys[kBlockThreads] is free for the bound
  __shared__ uint32_t wave_totals[kBlockThreads / kWaveLanes];
  const uint32_t row = blockIdx.x / units_out, unit = blockIdx.x - row * units_out;
  uint32_t hi[kE], lo[kE];
  if constexpr (kFromLists) {
    const uint32_t first_list = unit * fan;
    const uint32_t taken = min(fan, units_in - first_list) * a.count;
    const uint64_t *source = in_lists + ((size_t)row * units_in + first_list) * a.count;
#pragma unroll
    for (int j = 0; j < kE; ++j) {
      const uint32_t i = threadIdx.x + j * kBlockThreads;
      const uint64_t key = source[min(i, taken - 1)];  // an unconditional load, clamped
      hi[j] = i < taken ? (uint32_t)(key >> 32) : 0;
      lo[j] = i < taken ? (uint32_t)key : 0;
    }
  } else {
    const uint32_t first = unit * (kBlockThreads * kE);
    const int64_t base = row_base(a, row, kSize);
    if constexpr (kVector) {
      static_assert(kE % kVec == 0, "whole vectors per thread");
      // Every load is issued before the first key is made: addresses past the row's end are
      // clamped to its last vector (a load inside a branch would wait for itself there).
      const u32x4 *vectors = reinterpret_cast<const u32x4 *>(x + base);
      const uint32_t last_vector = a.width / kVec - 1;
      u32x4 raw[kE / kVec];
#pragma unroll
      for (int v = 0; v < kE / kVec; ++v) {
        const uint32_t vector = first / kVec + threadIdx.x + v * kBlockThreads;
        raw[v] = __builtin_nontemporal_load(vectors + min(vector, last_vector));
      }
#pragma unroll
      for (int v = 0; v < kE / kVec; ++v) {
        const uint32_t element = first + (threadIdx.x + v * kBlockThreads) * kVec;
        const bool inside = element < a.width;
        uint32_t bits[kVec];
        vector_bits<T>(raw[v], bits);
#pragma unroll
        for (int j = 0; j < kVec; ++j) {
          hi[v * kVec + j] = inside ? ordered_bits<T>(bits[j], largest != 0) : 0;
          lo[v * kVec + j] = inside ? ~(element + j) : 0;
        }
      }
    } else {
      const int64_t step = a.dense_last ? kSize : a.strides[a.axis];
      const uint32_t last = a.width - 1;
      uint32_t bits[kE];
#pragma unroll
      for (int j = 0; j < kE; ++j) {
        const uint32_t element = first + threadIdx.x + j * kBlockThreads;
        bits[j] = load_bits<T, kBytewise>(x + base + (int64_t)min(element, last) * step);
      }
#pragma unroll
      for (int j = 0; j < kE; ++j) {
        const uint32_t element = first + threadIdx.x + j * kBlockThreads;
        const bool inside = element < a.width;
        hi[j] = inside ? ordered_bits<T>(bits[j], largest != 0) : 0;
        lo[j] = inside ? ~element : 0;
      }
    }
  }
  auto key_of = [&](int j) { return ((uint64_t)hi[j] << 32) | lo[j]; };

  // A lower bound of the count-th largest ordered value: the count-th largest of the 256 thread
  // maxima (at least `count` keys reach it).  Each wave sorts its 64 maxima in registers (bitonic
  // network over lane exchanges), the four sorted runs meet in LDS, and every thread finds the
  // rank of its maximum among all 256 with three binary searches; ties rank by wave, so exactly
  // one thread has rank count - 1.  Everything whose ordered value reaches that bound is a
  // candidate: one 32-bit comparison per key.  A bound of 0 (fewer than `count` threads hold a
  // number) makes every key a candidate.
  uint32_t *maxima = reinterpret_cast<uint32_t *>(keys);
  uint32_t best = 0;
#pragma unroll
  for (int j = 0; j < kE; ++j) best = max(best, hi[j]);
  const uint32_t lane = threadIdx.x % kWaveLanes, wave = threadIdx.x / kWaveLanes;
#pragma unroll
  for (uint32_t size = 2; size <= kWaveLanes; size <<= 1) {
#pragma unroll
    for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
      const uint32_t other = __shfl_xor(best, stride, kWaveLanes);
      const bool descending = (lane & size) == 0;       // direction of this lane's run
      const bool lower_lane = (lane & stride) == 0;     // the lane that keeps the run's front value
      best = (lower_lane == descending) ? max(best, other) : min(best, other);
    }
  }
  maxima[threadIdx.x] = best;  // four descending runs of 64
  __syncthreads();
  {
    uint32_t rank = lane;  // larger values of the own run come first
#pragma unroll
    for (uint32_t w = 0; w < kBlockThreads / kWaveLanes; ++w) {
      if (w == wave) continue;
      // values of run w that precede `best`: strictly larger ones, and equal ones of earlier waves
      const uint32_t *run = maxima + w * kWaveLanes;
      uint32_t low = 0, high = kWaveLanes;  // first position whose value does not precede
      while (low < high) {
        const uint32_t mid = (low + high) >> 1;
        const uint32_t value = run[mid];
        const bool precedes = value > best || (value == best && w < wave);
        if (precedes) low = mid + 1;
        else high = mid;
      }
      rank += low;
    }
    if (rank == a.count - 1) maxima[kBlockThreads] = best;
  }
  __syncthreads();
  const uint32_t bound_hi = maxima[kBlockThreads];
  __syncthreads();
  uint32_t reach = 0, total;
  if (bound_hi != 0) {
#pragma unroll
    for (int j = 0; j < kE; ++j) reach += hi[j] >= bound_hi ? 1u : 0u;
  } else {
#pragma unroll
    for (int j = 0; j < kE; ++j) reach += (hi[j] | lo[j]) != 0 ? 1u : 0u;
  }
  uint32_t position = block_exclusive_scan(reach, wave_totals, &total);
  uint64_t exact = 0;  // nonzero: candidates are the keys >= exact instead
  if (total > kTile) {
    // The exact count-th largest key, one bit at a time: the largest t with >= count keys >= t.
    for (int bit = 63; bit >= 0; --bit) {
      const uint64_t trial = exact | (1ull << bit);
      uint32_t at_least = 0, sum;
#pragma unroll
      for (int j = 0; j < kE; ++j) at_least += key_of(j) >= trial ? 1u : 0u;
      block_exclusive_scan(at_least, wave_totals, &sum);
      if (sum >= a.count) exact = trial;
    }
    if (exact == 0) exact = 1;
    reach = 0;
#pragma unroll
    for (int j = 0; j < kE; ++j) reach += key_of(j) >= exact ? 1u : 0u;
    position = block_exclusive_scan(reach, wave_totals, &total);  // total == count: keys are unique
  }
  auto candidate = [&](int j) {
    if (exact != 0) return key_of(j) >= exact;
    return bound_hi != 0 ? hi[j] >= bound_hi : (hi[j] | lo[j]) != 0;
  };
  constexpr uint32_t kRanked = kTile / 2;  // candidates in keys[0, kRanked), ranked output above
  if (total <= kRanked / 2) {
    // Few candidates (the usual case): place each by counting the candidates above it.
    for (uint32_t i = threadIdx.x; i < a.count; i += kBlockThreads) keys[kRanked + i] = 0;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kE; ++j)
      if (candidate(j)) keys[position++] = key_of(j);
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < total; i += kBlockThreads) {
      const uint64_t key = keys[i];
      uint32_t above = 0;
#pragma unroll 8
      for (uint32_t other = 0; other < total; ++other) above += keys[other] > key ? 1u : 0u;
      if (above < a.count) keys[kRanked + above] = key;
    }
    __syncthreads();
    emit<T, kBytewise, kFinal>(keys + kRanked, a, row, x, values, indices,
                               out_lists + ((size_t)row * units_out + unit) * a.count);
    return;
  }
  uint32_t sort_n = 64;
  while (sort_n < kTile && (sort_n < total || sort_n < a.count)) sort_n <<= 1;
  for (uint32_t i = threadIdx.x; i < sort_n; i += kBlockThreads) keys[i] = 0;
  __syncthreads();
#pragma unroll
  for (int j = 0; j < kE; ++j)
    if (candidate(j) && position < kTile) keys[position++] = key_of(j);  // the guard never binds
  sort_descending(keys, sort_n);
  emit<T, kBytewise, kFinal>(keys, a, row, x, values, indices,
                             out_lists + ((size_t)row * units_out + unit) * a.count);
}

template <class T, int kE, bool kBytewise>
void select_tiles_launch(const TopKParams &p, const Addressing &a, const char *in, void *values,
                         int32_t *indices, uint64_t *lists, bool vector, hipStream_t s) {
  const dim3 grid(p.rows * p.tiles), block(kBlockThreads);
  const uint32_t largest = p.largest ? 1u : 0u;
  const bool final = p.tiles == 1;
#define HYLE_SELECT(VEC, BYTES, FINAL)                                                                   \
  hipLaunchKernelGGL((topk_select<T, kE, false, VEC, BYTES, FINAL>), grid, block, 0, s, in, values, indices, \
                     static_cast<const uint64_t *>(nullptr), lists, a, p.tiles, 1u, p.tiles, largest)
  if (vector) {
    if (final) HYLE_SELECT(true, false, true);
    else HYLE_SELECT(true, false, false);
  } else {
    if (final) HYLE_SELECT(false, kBytewise, true);
    else HYLE_SELECT(false, kBytewise, false);
  }
#undef HYLE_SELECT
}

template <class T, int kE, bool kBytewise>
void select_lists_launch(const TopKParams &p, const Addressing &a, const char *in, void *values,
                         int32_t *indices, const uint64_t *from, uint64_t *to, uint32_t lists, uint32_t fan,
                         uint32_t out, hipStream_t s) {
  const dim3 grid(p.rows * out), block(kBlockThreads);
  if (out == 1)
    hipLaunchKernelGGL((topk_select<T, kE, true, false, kBytewise, true>), grid, block, 0, s, in, values,
                       indices, from, to, a, lists, fan, out, 1u);
  else
    hipLaunchKernelGGL((topk_select<T, kE, true, false, kBytewise, false>), grid, block, 0, s, in, values,
                       indices, from, to, a, lists, fan, out, 1u);
}

uint32_t pow2_at_least(uint32_t n, uint32_t floor) {
  uint32_t p = floor;
  while (p < n) p <<= 1;
  return p;
}

template <class T, bool kBytewise>
hipError_t run(const TopKParams &p, const void *x, void *values, int32_t *indices, void *workspace,
               bool vector, hipStream_t s) {
  Addressing a{};
  a.width = p.width;
  a.inner = p.inner;
  a.count = p.count;
  a.dense_last = p.dense_last ? 1u : 0u;
  a.rank = p.rank;
  a.axis = p.axis;
  for (int d = 0; d < p.rank; ++d) {
    a.dims[d] = p.dims[d];
    a.strides[d] = p.strides[d];
  }
  const char *in = static_cast<const char *>(x);
  uint64_t *lists_a = static_cast<uint64_t *>(workspace);
  uint64_t *lists_b = lists_a + (size_t)p.rows * p.tiles * p.count;
  const uint32_t largest = p.largest ? 1u : 0u;
  const uint32_t tile_n = pow2_at_least(std::min(p.width, kTile), 64);
  const dim3 block(kBlockThreads);
  vector = vector && p.dense_last && p.width % KeyTraits<T>::kVec == 0;
  if (p.select) {
    if (p.tile_elements == kBlockThreads * 64)
      select_tiles_launch<T, 64, kBytewise>(p, a, in, values, indices, lists_a, vector, s);
    else if (p.tile_elements == kBlockThreads * 32)
      select_tiles_launch<T, 32, kBytewise>(p, a, in, values, indices, lists_a, vector, s);
    else
      select_tiles_launch<T, 8, kBytewise>(p, a, in, values, indices, lists_a, vector, s);
    uint32_t lists = p.tiles;
    uint64_t *from = lists_a, *to = lists_b;
    while (lists > 1) {
      const uint32_t out = (lists + p.fan - 1) / p.fan;
      if (p.fan * p.count > kBlockThreads * 8)
        select_lists_launch<T, 32, kBytewise>(p, a, in, values, indices, from, to, lists, p.fan, out, s);
      else
        select_lists_launch<T, 8, kBytewise>(p, a, in, values, indices, from, to, lists, p.fan, out, s);
      std::swap(from, to);
      lists = out;
    }
    return hipGetLastError();
  }
  if (p.runs && p.tiles > 1) {
    // whole tiles sorted (every key kept), then runs merged in pairs until one is left per row
    Addressing whole = a;
    whole.count = kTile;
    uint64_t *from = lists_a, *to = lists_a + (size_t)p.rows * p.tiles * kTile;
    if (vector)
      hipLaunchKernelGGL((topk_tiles<T, true, false, false>), dim3(p.rows * p.tiles), block, 0, s, in, values, indices,
                         from, whole, p.tiles, kTile, largest);
    else
      hipLaunchKernelGGL((topk_tiles<T, false, kBytewise, false>), dim3(p.rows * p.tiles), block, 0, s, in, values,
                         indices, from, whole, p.tiles, kTile, largest);
    const uint32_t limit = (p.count + kTile - 1) / kTile * kTile;  // no run needs more keys than this
    uint32_t runs = p.tiles, run_keys = kTile;
    while (runs > 1) {
      const uint32_t runs_out = (runs + 1) / 2, out_keys = std::min(2 * run_keys, limit);
      hipLaunchKernelGGL(topk_merge_runs, dim3(p.rows * runs_out * (out_keys / kTile)), block, 0, s, from, to, runs,
                         run_keys, runs_out, out_keys);
      std::swap(from, to);
      runs = runs_out;
      run_keys = out_keys;
    }
    const uint32_t blocks_per_row = (p.count + kBlockThreads - 1) / kBlockThreads;
    hipLaunchKernelGGL((topk_emit_run<T, kBytewise>), dim3(p.rows * blocks_per_row), block, 0, s, in, values, indices,
                       from, a, run_keys, blocks_per_row);
    return hipGetLastError();
  }
  if (p.tiles == 1) {
    if (vector)
      hipLaunchKernelGGL((topk_tiles<T, true, false, true>), dim3(p.rows), block, 0, s, in, values, indices,
                         lists_a, a, 1u, tile_n, largest);
    else
      hipLaunchKernelGGL((topk_tiles<T, false, kBytewise, true>), dim3(p.rows), block, 0, s, in, values,
                         indices, lists_a, a, 1u, tile_n, largest);
    return hipGetLastError();
  }
  if (vector)
    hipLaunchKernelGGL((topk_tiles<T, true, false, false>), dim3(p.rows * p.tiles), block, 0, s, in, values,
                       indices, lists_a, a, p.tiles, kTile, largest);
  else
    hipLaunchKernelGGL((topk_tiles<T, false, kBytewise, false>), dim3(p.rows * p.tiles), block, 0, s, in,
                       values, indices, lists_a, a, p.tiles, kTile, largest);
  uint32_t lists = p.tiles;
  uint64_t *from = lists_a, *to = lists_b;
  while (lists > 1) {
    const uint32_t out = (lists + p.fan - 1) / p.fan;
    const uint32_t sort_n = pow2_at_least(std::min(lists, p.fan) * p.count, 64);
    if (out == 1)
      hipLaunchKernelGGL((topk_merge<T, kBytewise, true>), dim3(p.rows), block, 0, s, in, values, indices, from,
                         to, a, lists, p.fan, 1u, sort_n);
    else
      hipLaunchKernelGGL((topk_merge<T, kBytewise, false>), dim3(p.rows * out), block, 0, s, in, values,
                         indices, from, to, a, lists, p.fan, out, sort_n);
    std::swap(from, to);
    lists = out;
  }
  return hipGetLastError();
}

}  // namespace

uint32_t topk_max_count() { return kTile / 2; }  // above it: sorted runs merged in pairs

void topk_plan(TopKParams *p) {
  p->select = p->count <= kSelectMax;
  if (p->select) {
    // 16384- or 8192-element tiles for long rows (64 or 32 keys per thread: the per-block work of
    // finding the bound is paid once per tile), 2048 otherwise; merges take as many
    // lists as 8192 keys hold (2048 when that already covers every tile of a row).
    p->tile_elements = p->width > 8 * kTile ? kBlockThreads * 64
                                            : (p->width > kTile ? kBlockThreads * 32 : kBlockThreads * 8);
    p->tiles = (p->width + p->tile_elements - 1) / p->tile_elements;
    p->fan = (p->tiles * p->count <= kBlockThreads * 8 ? kBlockThreads * 8 : kBlockThreads * 32) / p->count;
  } else {
    p->tile_elements = kTile;
    p->tiles = (p->width + kTile - 1) / kTile;
    p->runs = p->count > kTile / 2;
    p->fan = p->runs ? 2 : kTile / p->count;  // >= 2 for count <= kTile / 2
  }
  p->dispatches = 1;
  p->workspace_bytes = 0;
  if (p->runs && p->tiles > 1) {
    // sorted tiles, merges of pairs of runs, one dispatch for the outputs; two buffers of whole tiles
    for (uint32_t runs = p->tiles; runs > 1; runs = (runs + 1) / 2) ++p->dispatches;
    ++p->dispatches;
    p->workspace_bytes = 2 * (size_t)p->rows * p->tiles * kTile * sizeof(uint64_t);
    return;
  }
  if (p->tiles > 1) {
    uint32_t lists = p->tiles;
    while (lists > 1) {
      lists = (lists + p->fan - 1) / p->fan;
      ++p->dispatches;
    }
    const size_t first = (size_t)p->rows * p->tiles * p->count;
    const size_t second = (size_t)p->rows * ((p->tiles + p->fan - 1) / p->fan) * p->count;
    p->workspace_bytes = (first + second) * sizeof(uint64_t);
  }
}

hipError_t launch_topk(Elem type, const TopKParams &p, const void *x, void *values, int32_t *indices,
                       void *workspace, bool input_vector_aligned, hipStream_t stream) {
  if (p.rows == 0 || p.count == 0) return hipSuccess;
  if (p.integer)
    return p.bytewise ? run<I32, true>(p, x, values, indices, workspace, false, stream)
                      : run<I32, false>(p, x, values, indices, workspace, input_vector_aligned, stream);
  switch (type) {
    case Elem::kF32:
      return p.bytewise ? run<F32, true>(p, x, values, indices, workspace, false, stream)
                        : run<F32, false>(p, x, values, indices, workspace, input_vector_aligned, stream);
    case Elem::kF16:
      return p.bytewise ? run<F16, true>(p, x, values, indices, workspace, false, stream)
                        : run<F16, false>(p, x, values, indices, workspace, input_vector_aligned, stream);
    case Elem::kBF16:
      return p.bytewise ? run<BF16, true>(p, x, values, indices, workspace, false, stream)
                        : run<BF16, false>(p, x, values, indices, workspace, input_vector_aligned, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace hyle_hip
