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
// block therefore *selects* instead (select_tile): in the float domain, a bound that at least k
// elements of the tile reach comes from the threads' maxima; one comparison per element finds the
// few that reach it -- for unordered data a little more than k -- and only those become keys, in
// LDS, ranked by counting.  The lists of the tiles of a row meet in one more dispatch
// (topk_rank_lists) that bounds and ranks the same way.  Ordered data, NaN-heavy tiles and int32
// take a general form with ordered keys for every element.
#include <algorithm>
#include <type_traits>

#include "device_common.h"
#include "kernels.h"

namespace hyle_hip {
namespace {

constexpr uint32_t kTile = 2048;  // keys one block sorts: 16 KiB of LDS

struct Addressing {
  uint32_t width, inner, count;  // extent of the axis, elements after it, k
  uint32_t largest;              // 1: largest first
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
// The inverse of ordered_bits where it has one: false for a NaN and for a zero.
template <class T> __device__ __forceinline__ bool storage_bits_of(uint32_t ordered, bool largest, uint32_t *bits) {
  if constexpr (std::is_same<T, I32>::value) {
    *bits = (largest ? ordered : ~ordered) ^ 0x80000000u;
    return true;
  } else {
    if (ordered == 0) return false;  // NaN
    const uint32_t up = largest ? ordered : ~ordered;
    const uint32_t wide = (up & 0x80000000u) ? up ^ 0x80000000u : ~up;
    if (wide == 0) return false;  // +0 stands for both zeros
    if constexpr (KeyTraits<T>::kSize == 4) {
      *bits = wide;
    } else {
      uint16_t narrow;  // exact: the value came from this storage type
      Traits<T>::store(&narrow, 0, bits_f32(wide));
      *bits = narrow;
    }
    return true;
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
    for (uint32_t j = threadIdx.x; j < a.count; j += blockDim.x) {
      // a list always holds `count` elements of the row here; the clamp only keeps a corrupted
      // workspace from turning into a wild address
      const uint32_t index = min(~(uint32_t)keys[j], a.width - 1);
      // The ordered half of the key gives the storage bits back, except where it folded several
      // patterns into one: zeros (the sign) and NaNs (everything).  Only those are read again.
      uint32_t bits;
      if (!storage_bits_of<T>((uint32_t)(keys[j] >> 32), a.largest != 0, &bits))
        bits = load_bits<T, kBytewise>(x + base + (int64_t)index * step);
      const size_t out = ((size_t)outer * a.count + j) * a.inner + position;
      if constexpr (kSize == 4) static_cast<uint32_t *>(values)[out] = bits;
      else static_cast<uint16_t *>(values)[out] = (uint16_t)bits;
      indices[out] = (int32_t)index;
    }
  } else {
    for (uint32_t j = threadIdx.x; j < a.count; j += blockDim.x) list[j] = keys[j];
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

// ---- wave-local pieces of the select route ------------------------------------------------------
// The value of lane ^ kStride: strides below 16 stay inside a DPP row (stride 4 is a half-row
// mirror followed by a quad reversal), 16 goes through the swizzle unit, 32 through a permute.
template <int kStride> __device__ __forceinline__ int lane_xor(int v) {
  if constexpr (kStride == 1) return dpp_move<kDppSwap1>(v);
  else if constexpr (kStride == 2) return dpp_move<kDppSwap2>(v);
  else if constexpr (kStride == 4) return dpp_move<0x1B>(dpp_move<kDppHalfMirror>(v));  // quad_perm [3,2,1,0]
  else if constexpr (kStride == 8) return dpp_move<0x128>(v);                            // row_ror:8
  else if constexpr (kStride == 16) return __builtin_amdgcn_ds_swizzle(v, 0x401F);       // xor 16 within 32 lanes
  else return __shfl_xor(v, 32, kWaveLanes);
}
template <int kStride> __device__ __forceinline__ uint64_t lane_xor(uint64_t v) {
  return ((uint64_t)(uint32_t)lane_xor<kStride>((int)(uint32_t)(v >> 32)) << 32) |
         (uint32_t)lane_xor<kStride>((int)(uint32_t)v);
}
__device__ __forceinline__ uint64_t as_lane_word(uint64_t v) { return v; }
__device__ __forceinline__ void from_lane_word(uint64_t w, uint64_t *v) { *v = w; }
__device__ __forceinline__ int as_lane_word(float v) { return __float_as_int(v); }
__device__ __forceinline__ int as_lane_word(uint32_t v) { return (int)v; }
__device__ __forceinline__ void from_lane_word(int w, float *v) { *v = __int_as_float(w); }
__device__ __forceinline__ void from_lane_word(int w, uint32_t *v) { *v = (uint32_t)w; }
// One compare-exchange of a bitonic network: the lane that keeps the front of a descending run
// takes the other value when that is larger, its partner when it is smaller (equal values may
// go either way).  One comparison, the lane's role folded into the mask.
template <int kSize, int kStride, class V> __device__ __forceinline__ V sort_step(V v, uint32_t lane) {
  V other;
  from_lane_word(lane_xor<kStride>(as_lane_word(v)), &other);
  const bool descending = (lane & kSize) == 0;    // direction of this lane's run
  const bool lower_lane = (lane & kStride) == 0;  // the lane that keeps the run's front value
  const bool wants_smaller = lower_lane != descending;
  return ((other > v) != wants_smaller) ? other : v;
}
template <int kSize, int kStride, class V> __device__ __forceinline__ V sort_steps(V v, uint32_t lane) {
  v = sort_step<kSize, kStride>(v, lane);
  if constexpr (kStride > 1) v = sort_steps<kSize, kStride / 2>(v, lane);
  return v;
}
// The wave's 64 values (floats: no NaN among them) in descending lane order.
template <class V> __device__ __forceinline__ V wave_sort_descending(V v, uint32_t lane) {
  v = sort_steps<2, 1>(v, lane);
  v = sort_steps<4, 2>(v, lane);
  v = sort_steps<8, 4>(v, lane);
  v = sort_steps<16, 8>(v, lane);
  v = sort_steps<32, 16>(v, lane);
  v = sort_steps<64, 32>(v, lane);  // lane & 64 == 0 for every lane: one descending run
  return v;
}

// Storage bits with the sign flipped when the smallest are wanted, so that "better" is always
// "larger as a float"; the pattern of a quiet NaN stands for "no element".
template <class T> constexpr uint32_t kSignBit = KeyTraits<T>::kSize == 4 ? 0x80000000u : 0x8000u;
template <class T> constexpr uint32_t kNoElement = KeyTraits<T>::kSize == 4 ? 0x7FC00000u : (std::is_same<T, F16>::value ? 0x7E00u : 0x7FC0u);

// LDS of the select route, in keys: wave-private candidate segments, the compacted candidates,
// the ranked result.
constexpr uint32_t kSegment = 128;                        // candidates one wave may collect
constexpr uint32_t kCompact = 4 * kSegment;               // keys[kCompact ...): all candidates, contiguous
constexpr uint32_t kRanked = kTile / 2;                   // keys[kRanked ...): the `count` best, descending
constexpr uint32_t kFewCandidates = 256;                  // above it the keys are sorted, not ranked

// keys[from, from + total) unique and unordered, followed by kParts - 1 zero keys -> the `count`
// largest, descending, in keys[kRanked ...).  kParts neighbouring threads share a candidate: each
// counts its share of the keys above it (the zeros let every share run the same number of
// steps).  Needs total >= count (every rank below count is then written) and a barrier before
// and after.
template <int kThreads, int kParts>
__device__ __forceinline__ void rank_candidates(uint64_t *keys, uint32_t from, uint32_t total, uint32_t count) {
  static_assert(kParts == 4 || kParts == 16, "a quad or a DPP row per candidate");
  const uint32_t part = threadIdx.x % kParts, steps = (total + kParts - 1) / kParts;
  const uint64_t *candidates = keys + from;
  for (uint32_t first = 0; first < total; first += kThreads / kParts) {
    const uint32_t mine = first + threadIdx.x / kParts;
    const uint64_t key = candidates[min(mine, total - 1)];
    uint32_t above = 0;
#pragma unroll 8
    for (uint32_t step = 0; step < steps; ++step) above += candidates[kParts * step + part] > key ? 1u : 0u;
    above += (uint32_t)dpp_move<kDppSwap1>((int)above);
    above += (uint32_t)dpp_move<kDppSwap2>((int)above);
    if constexpr (kParts == 16) {
      above += (uint32_t)dpp_move<kDppHalfMirror>((int)above);
      above += (uint32_t)dpp_move<kDppRowMirror>((int)above);
    }
    if (mine < total && part == 0 && above < count) keys[kRanked + above] = key;
  }
}

struct SelectShared {
  uint64_t keys[kTile];  // kBlockThreads < kTile / 2: keys[kBlockThreads] is free for the general form's bound
  uint32_t wave_totals[kBlockThreads / kWaveLanes];
  float wave_bound[kBlockThreads / kWaveLanes];
  uint32_t wave_count[kBlockThreads / kWaveLanes];
};

// The `count` best of one tile of 256 * kE elements of `row`, starting at element `first`, whose
// storage bits the threads hold in `bits` (slot j of a thread is element_of(j); loads past the
// row's end were clamped): values and indices (kFinal) or a descending list of keys.  Called by
// every thread of the block; ends with the block's LDS free again.
//
// Float types first try in the float domain: a thread's maximum over its elements ignores NaNs
// (fmaxf), each wave sorts its 64 thread maxima in registers, and the smallest of the four waves'
// ceil(count / 4)-th largest is a bound that at least `count` elements of the tile reach.  Each
// wave then walks its elements once more: one comparison per element, and for the few that reach
// the bound -- for unordered data a little more than `count` in the tile -- a 64-bit key goes to
// the wave's own segment of LDS, placed by the comparison mask alone (no atomics).  The segments
// are packed together and ranked by counting.  When the bound is not a number above -inf (too few
// numbers in some wave: NaNs must then be ranked too), when too many elements reach it (ordered
// data), and for int32, the tile takes the general form: ordered 32-bit values for every element,
// the count-th largest of the 256 thread maxima as the bound, the exact count-th key bit by bit
// if need be.
template <class T, int kE, bool kVector, bool kBytewise, bool kFinal>
__device__ __forceinline__ void select_tile(uint32_t (&bits)[kE], uint32_t first, const Addressing &a, uint32_t row,
                                            uint32_t largest, const char *x, void *values, int32_t *indices,
                                            uint64_t *list, SelectShared &shared) {
  constexpr int kVec = KeyTraits<T>::kVec;
  constexpr bool kFloat = !std::is_same<T, I32>::value;
  uint64_t *keys = shared.keys;
  const uint32_t lane = threadIdx.x % kWaveLanes, wave = threadIdx.x / kWaveLanes;
  auto element_of = [&](int j) -> uint32_t {
    if constexpr (kVector) return first + (threadIdx.x + (j / kVec) * kBlockThreads) * kVec + (j % kVec);
    else return first + threadIdx.x + j * kBlockThreads;
  };
  const bool whole = first + kBlockThreads * kE <= a.width;  // no slot lies past the row's end

  if constexpr (kFloat) {
    // storage bits with the sign flipped when the smallest are wanted, so that "better" is
    // "larger as a float"; a quiet NaN stands for "no element"
    const uint32_t flip = largest != 0 ? 0u : kSignBit<T>;
    if (!whole) {
#pragma unroll
      for (int j = 0; j < kE; ++j) bits[j] = element_of(j) < a.width ? bits[j] : kNoElement<T>;
    }
    if (flip != 0) {
#pragma unroll
      for (int j = 0; j < kE; ++j) bits[j] ^= flip;
    }
    float best = -INFINITY;
#pragma unroll
    for (int j = 0; j < kE; ++j) best = fmaxf(best, bits_value<T>(bits[j]));
    best = wave_sort_descending(best, lane);
    const uint32_t per_wave = (a.count + 3) / 4;  // <= 64: the select route serves counts up to 256
    const float wave_share = __shfl(best, (int)per_wave - 1, kWaveLanes);
    if (lane == 0) shared.wave_bound[wave] = wave_share;
    __syncthreads();
    const float bound = fminf(fminf(shared.wave_bound[0], shared.wave_bound[1]),
                              fminf(shared.wave_bound[2], shared.wave_bound[3]));
    bool done = false;
    if (bound > -INFINITY) {  // the same for every thread of the block
      uint64_t *segment = keys + wave * kSegment;
      uint32_t collected = 0;  // the same in every lane of the wave
#pragma unroll
      for (int j = 0; j < kE; ++j) {
        const bool reaches = bits_value<T>(bits[j]) >= bound;
        const uint64_t mask = __ballot(reaches);
        if (mask != 0) {
          const uint32_t place = collected + __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32),
                                                                     __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
          if (reaches && place < kSegment)
            segment[place] = make_key<T>(bits[j] ^ flip, element_of(j), largest != 0);
          collected += (uint32_t)__popcll(mask);
        }
      }
      if (lane == 0) shared.wave_count[wave] = collected;
      __syncthreads();
      uint32_t before = 0, total = 0;
      bool fits = true;
#pragma unroll
      for (uint32_t w = 0; w < kBlockThreads / kWaveLanes; ++w) {
        const uint32_t c = shared.wave_count[w];
        if (w < wave) before += c;
        total += c;
        fits = fits && c <= kSegment;
      }
      if (fits && total <= kFewCandidates) {  // total >= count: the bound's guarantee
        for (uint32_t i = lane; i < collected; i += kWaveLanes) keys[kCompact + before + i] = segment[i];
        if (threadIdx.x < 3) keys[kCompact + total + threadIdx.x] = 0;
        __syncthreads();
        rank_candidates<kBlockThreads, 4>(keys, kCompact, total, a.count);
        __syncthreads();
        emit<T, kBytewise, kFinal>(keys + kRanked, a, row, x, values, indices, list);
        done = true;
      }
    }
    __syncthreads();  // LDS is free again (or about to be reused by the general form)
    if (done) return;
    if (flip != 0) {
#pragma unroll
      for (int j = 0; j < kE; ++j) bits[j] ^= flip;  // storage bits again; "no element" is told by the index below
    }
  }

  // ---- the general form ----------------------------------------------------------------------------
  // A thread keeps its kE keys as two words, hi (ordered value) and lo (~index, recomputed from
  // the slot number); an empty slot is hi = lo = 0.
  uint32_t(&hi)[kE] = bits;  // converted in place: the storage bits are not needed again
#pragma unroll
  for (int j = 0; j < kE; ++j) hi[j] = element_of(j) < a.width ? ordered_bits<T>(bits[j], largest != 0) : 0;
  auto lo_of = [&](int j) -> uint32_t { return element_of(j) < a.width ? ~element_of(j) : 0u; };
  auto key_of = [&](int j) { return ((uint64_t)hi[j] << 32) | lo_of(j); };

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
    for (int j = 0; j < kE; ++j) reach += (hi[j] | lo_of(j)) != 0 ? 1u : 0u;
  }
  uint32_t position = block_exclusive_scan(reach, shared.wave_totals, &total);
  uint64_t exact = 0;  // nonzero: candidates are the keys >= exact instead
  if (total > kTile) {
    // The exact count-th largest key, one bit at a time: the largest t with >= count keys >= t.
    for (int bit = 63; bit >= 0; --bit) {
      const uint64_t trial = exact | (1ull << bit);
      uint32_t at_least = 0, sum;
#pragma unroll
      for (int j = 0; j < kE; ++j) at_least += key_of(j) >= trial ? 1u : 0u;
      block_exclusive_scan(at_least, shared.wave_totals, &sum);
      if (sum >= a.count) exact = trial;
    }
    if (exact == 0) exact = 1;
    reach = 0;
#pragma unroll
    for (int j = 0; j < kE; ++j) reach += key_of(j) >= exact ? 1u : 0u;
    position = block_exclusive_scan(reach, shared.wave_totals, &total);  // total == count: keys are unique
  }
  auto candidate = [&](int j) {
    if (exact != 0) return key_of(j) >= exact;
    return bound_hi != 0 ? hi[j] >= bound_hi : (hi[j] | lo_of(j)) != 0;
  };
  if (total <= kFewCandidates && total >= a.count) {
    // Few candidates: place each by counting the candidates above it.
#pragma unroll
    for (int j = 0; j < kE; ++j)
      if (candidate(j)) keys[position++] = key_of(j);
    if (threadIdx.x < 3) keys[total + threadIdx.x] = 0;
    __syncthreads();
    rank_candidates<kBlockThreads, 4>(keys, 0, total, a.count);
    __syncthreads();
    emit<T, kBytewise, kFinal>(keys + kRanked, a, row, x, values, indices, list);
    __syncthreads();
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
  emit<T, kBytewise, kFinal>(keys, a, row, x, values, indices, list);
  __syncthreads();
}

// One block per (row, tile of 256 * kE elements); each tile leaves its own list (or, for a row of
// one tile, the outputs).  Measured on MI355X for TopK(64) over [64, 151936] f32: tiles of 8192
// elements 15.3 us, of 16384 (64 registers of elements per thread) 16.3 us; two tiles per block
// with every load issued up front, so that one tile is selected while the next arrives, 17.9 us.
template <class T, int kE, bool kVector, bool kBytewise, bool kFinal>
__global__ __launch_bounds__(kBlockThreads) void topk_select(const char *x, void *values, int32_t *indices,
                                                             uint64_t *out_lists, Addressing a, uint32_t tiles,
                                                             uint32_t largest) {
  constexpr int kSize = KeyTraits<T>::kSize;
  constexpr int kVec = KeyTraits<T>::kVec;
  __shared__ SelectShared shared;
  const uint32_t row = blockIdx.x / tiles, tile = blockIdx.x - row * tiles;
  const uint32_t first = tile * (kBlockThreads * kE);
  const int64_t base = row_base(a, row, kSize);
  // Every load is issued before the first value is looked at: addresses past the row's end are
  // clamped to its last vector or element (a load inside a branch would wait for itself there).
  uint32_t bits[kE];
  if constexpr (kVector) {
    static_assert(kE % kVec == 0, "whole vectors per thread");
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
      uint32_t piece[kVec];
      vector_bits<T>(raw[v], piece);
#pragma unroll
      for (int j = 0; j < kVec; ++j) bits[v * kVec + j] = piece[j];
    }
  } else {
    const int64_t step = a.dense_last ? kSize : a.strides[a.axis];
    const uint32_t last = a.width - 1;
#pragma unroll
    for (int j = 0; j < kE; ++j)
      bits[j] = load_bits<T, kBytewise>(x + base + (int64_t)min(first + threadIdx.x + j * kBlockThreads, last) * step);
  }
  select_tile<T, kE, kVector, kBytewise, kFinal>(bits, first, a, row, largest, x, values, indices,
                                                 out_lists + ((size_t)row * tiles + tile) * a.count, shared);
}

constexpr int kMergeThreads = 1024;  // one block per row: the work of a merge is latency, spread over 16 waves

template <class T, bool kBytewise, bool kFinal>
__global__ __launch_bounds__(kMergeThreads) void topk_rank_lists(const char *x, void *values, int32_t *indices,
                                                                 const uint64_t *in_lists, uint64_t *out_lists,
                                                                 Addressing a, uint32_t units_in, uint32_t fan,
                                                                 uint32_t units_out) {
  extern __shared__ uint64_t merged[];  // fan * count keys
  __shared__ uint64_t chosen[kTile];    // candidates in [0, kRanked), the ranked result above
  __shared__ uint32_t reached;
  __shared__ uint64_t bound_slot;
  const uint32_t row = blockIdx.x / units_out, unit = blockIdx.x - row * units_out;
  const uint32_t first_list = unit * fan;
  const uint32_t lists = min(fan, units_in - first_list), taken = lists * a.count;
  const uint64_t *source = in_lists + ((size_t)row * units_in + first_list) * a.count;
  uint64_t *ranked = chosen + kRanked;
  uint64_t *list = out_lists + ((size_t)row * units_out + unit) * a.count;
  for (uint32_t i = threadIdx.x; i < taken; i += kMergeThreads) merged[i] = source[i];
  for (uint32_t i = threadIdx.x; i < a.count; i += kMergeThreads) ranked[i] = 0;  // a short last tile leaves "no element" keys
  if (threadIdx.x == 0) reached = 0;
  __syncthreads();
  // The bound comes from samples of the lists.  A sample at place p of its list stands for the
  // keys above it down to the list's previous sample: p + 1 keys of that list reach it.  Walking
  // all samples from the largest down and adding those weights, the first sample at which the sum
  // reaches `count` is a bound that at least `count` keys reach.  Up to 64 samples -- up to eight
  // per list, placed around count / lists, where a list's share of the result ends on average --
  // are sorted with their weights in the registers of one wave, and only their ordered values are
  // compared (equal values of other indices come along).  A weak list (a row's short last tile)
  // sends weak samples and does not pull the bound down.  More than 64 lists: one sample per list
  // at the same place in each, ranked by counting.
  if (threadIdx.x == 0) bound_slot = 0;
  __syncthreads();
  if (lists <= kWaveLanes) {
    if (threadIdx.x < kWaveLanes) {
      uint32_t per_list = kWaveLanes / lists;
      per_list = per_list > 8 ? 8 : per_list;
      const uint32_t own_list = threadIdx.x / per_list, nth = threadIdx.x - own_list * per_list;
      // places: share * {0.4, 0.8, 1.2, 1.7, 2.4, 3.4, 5, 8}, stretched so that the last one used
      // is at least 2.5 shares deep; strictly increasing, inside the list
      const float factors[8] = {0.4f, 0.8f, 1.2f, 1.7f, 2.4f, 3.4f, 5.0f, 8.0f};
      const float stretch = factors[per_list - 1] < 2.5f ? 2.5f / factors[per_list - 1] : 1.0f;
      const float share = (float)a.count / (float)lists * stretch;
      uint32_t place = 0, previous = 0, weight = 0, value = 0;
      for (uint32_t i = 0; i <= nth; ++i) {
        const uint32_t wanted_place = (uint32_t)ceilf(share * factors[i]);
        previous = place;                                                  // keys before this sample's span
        place = wanted_place > previous ? wanted_place : previous + 1;     // place = p + 1
      }
      if (own_list < lists && place <= a.count) {
        weight = place - previous;
        value = (uint32_t)(merged[own_list * a.count + place - 1] >> 32);
      }
      // descending by value, the weight travelling with it
      uint64_t pair = ((uint64_t)value << 32) | weight;
      pair = wave_sort_descending(pair, threadIdx.x);
      uint32_t reached_by = (uint32_t)pair;
#pragma unroll
      for (int d = 1; d < kWaveLanes; d <<= 1) {
        const uint32_t other = __shfl_up(reached_by, d, kWaveLanes);
        if (threadIdx.x >= (uint32_t)d) reached_by += other;
      }
      const uint64_t enough = __ballot(reached_by >= a.count && (uint32_t)(pair >> 32) != 0);
      if (enough != 0 && threadIdx.x == (uint32_t)__ffsll((long long)enough) - 1) bound_slot = pair & 0xFFFFFFFF00000000ull;
    }
  } else {
    const uint32_t place = (a.count + lists - 1) / lists < a.count ? (a.count + lists - 1) / lists : a.count;
    const uint32_t wanted = (a.count + place - 1) / place;
    for (uint32_t own_list = threadIdx.x; own_list < lists; own_list += kMergeThreads) {
      const uint64_t key = merged[own_list * a.count + place - 1];
      uint32_t above = 0;
      for (uint32_t l = 0; l < lists; ++l) above += merged[l * a.count + place - 1] > key ? 1u : 0u;
      if (above == wanted - 1 && key != 0) bound_slot = key;  // keys are unique: at most one writer
    }
  }
  __syncthreads();
  const uint64_t bound = bound_slot;
  if (bound != 0) {  // 0: fewer real samples than the bound needs
    uint32_t reach = 0;
    for (uint32_t i = threadIdx.x; i < taken; i += kMergeThreads) reach += merged[i] >= bound ? 1u : 0u;
    uint32_t position = 0;
    if (reach != 0) position = atomicAdd(&reached, reach);
    __syncthreads();
    const uint32_t total = reached;  // >= count
    if (total <= kRanked - 16) {
      for (uint32_t i = threadIdx.x; i < taken; i += kMergeThreads)
        if (merged[i] >= bound) chosen[position++] = merged[i];
      if (threadIdx.x < 15) chosen[total + threadIdx.x] = 0;
      __syncthreads();
      rank_candidates<kMergeThreads, 16>(chosen, 0, total, a.count);
      __syncthreads();
      emit<T, kBytewise, kFinal>(ranked, a, row, x, values, indices, list);
      return;
    }
  }
  for (uint32_t i = threadIdx.x; i < taken; i += kMergeThreads) {
    const uint64_t key = merged[i];
    const uint32_t own = i / a.count;
    uint32_t rank = i - own * a.count;
    for (uint32_t l = 0; l < lists && rank < a.count; ++l) {
      if (l == own) continue;
      const uint64_t *other = merged + (size_t)l * a.count;
      uint32_t low = 0, high = a.count;  // first position whose key is not above `key`
      while (low < high) {
        const uint32_t mid = (low + high) >> 1;
        if (other[mid] > key) low = mid + 1;
        else high = mid;
      }
      rank += low;
    }
    if (rank < a.count && key != 0) ranked[rank] = key;
  }
  __syncthreads();
  emit<T, kBytewise, kFinal>(ranked, a, row, x, values, indices, list);
}

// Launch-shape labels: topk_<kernel>/<form>...
inline std::string access_word(bool vector, bool bytewise) { return vector ? "vector" : (bytewise ? "bytes" : "scalar"); }
template <int kE, bool kVector, bool kBytewise, bool kFinal> struct SelectTag {
  static std::string text() {
    return "topk_select/" + std::to_string(kE) + "x256/" + access_word(kVector, kBytewise) + (kFinal ? "/final" : "/lists");
  }
};
template <bool kBytewise, bool kFinal> struct RankListsTag {
  static std::string text() { return std::string("topk_rank_lists") + (kBytewise ? "/bytes" : "") + (kFinal ? "/final" : "/lists"); }
};
template <bool kVector, bool kBytewise, bool kFinal> struct TilesTag {
  static std::string text() { return "topk_tiles/" + access_word(kVector, kBytewise) + (kFinal ? "/final" : "/lists"); }
};
template <bool kBytewise, bool kFinal> struct MergeTag {
  static std::string text() { return std::string("topk_merge") + (kBytewise ? "/bytes" : "") + (kFinal ? "/final" : "/lists"); }
};
struct MergeRunsTag {
  static std::string text() { return "topk_merge_runs"; }
};
template <bool kBytewise> struct EmitRunTag {
  static std::string text() { return std::string("topk_emit_run") + (kBytewise ? "/bytes" : ""); }
};

template <class T, int kE, bool kBytewise>
void select_tiles_launch(const TopKParams &p, const Addressing &a, const char *in, void *values,
                         int32_t *indices, uint64_t *lists, bool vector, hipStream_t s) {
  const dim3 grid(p.rows * p.tiles), block(kBlockThreads);
  const uint32_t largest = p.largest ? 1u : 0u;
  const bool final = p.tiles == 1;
#define HYLE_SELECT(VEC, BYTES, FINAL)                                                                   \
  note_variant<SelectTag<kE, VEC, BYTES, FINAL>>();                                                         \
  hipLaunchKernelGGL((topk_select<T, kE, VEC, BYTES, FINAL>), grid, block, 0, s, in, values, indices, lists, a, \
                     p.tiles, largest)
  // tiles of 2048 elements are chosen only for rows that one of them covers (topk_plan): no lists there
  if (vector) {
    if (final) { HYLE_SELECT(true, false, true); }
    else if constexpr (kE != 8) { HYLE_SELECT(true, false, false); }
  } else {
    if (final) { HYLE_SELECT(false, kBytewise, true); }
    else if constexpr (kE != 8) { HYLE_SELECT(false, kBytewise, false); }
  }
#undef HYLE_SELECT
}

template <class T, bool kBytewise>
void rank_lists_launch(const TopKParams &p, const Addressing &a, const char *in, void *values, int32_t *indices,
                       const uint64_t *from, uint64_t *to, uint32_t lists, uint32_t fan, uint32_t out,
                       hipStream_t s) {
  const dim3 grid(p.rows * out), block(kMergeThreads);
  const size_t shared = (size_t)fan * p.count * sizeof(uint64_t);
  if (out == 1) {
    note_variant<RankListsTag<kBytewise, true>>();
    hipLaunchKernelGGL((topk_rank_lists<T, kBytewise, true>), grid, block, shared, s, in, values, indices, from, to,
                       a, lists, fan, out);
  } else {
    note_variant<RankListsTag<kBytewise, false>>();
    hipLaunchKernelGGL((topk_rank_lists<T, kBytewise, false>), grid, block, shared, s, in, values, indices, from,
                       to, a, lists, fan, out);
  }
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
  a.largest = p.largest ? 1u : 0u;
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
    if (p.tile_elements == kBlockThreads * 32)
      select_tiles_launch<T, 32, kBytewise>(p, a, in, values, indices, lists_a, vector, s);
    else
      select_tiles_launch<T, 8, kBytewise>(p, a, in, values, indices, lists_a, vector, s);
    uint32_t lists = p.tiles;
    uint64_t *from = lists_a, *to = lists_b;
    while (lists > 1) {
      const uint32_t out = (lists + p.fan - 1) / p.fan;
      rank_lists_launch<T, kBytewise>(p, a, in, values, indices, from, to, lists, p.fan, out, s);
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
    if (vector) {
      note_variant<TilesTag<true, false, false>>();
      hipLaunchKernelGGL((topk_tiles<T, true, false, false>), dim3(p.rows * p.tiles), block, 0, s, in, values, indices,
                         from, whole, p.tiles, kTile, largest);
    } else {
      note_variant<TilesTag<false, kBytewise, false>>();
      hipLaunchKernelGGL((topk_tiles<T, false, kBytewise, false>), dim3(p.rows * p.tiles), block, 0, s, in, values,
                         indices, from, whole, p.tiles, kTile, largest);
    }
    const uint32_t limit = (p.count + kTile - 1) / kTile * kTile;  // no run needs more keys than this
    uint32_t runs = p.tiles, run_keys = kTile;
    while (runs > 1) {
      const uint32_t runs_out = (runs + 1) / 2, out_keys = std::min(2 * run_keys, limit);
      note_variant<MergeRunsTag>();
      hipLaunchKernelGGL(topk_merge_runs, dim3(p.rows * runs_out * (out_keys / kTile)), block, 0, s, from, to, runs,
                         run_keys, runs_out, out_keys);
      std::swap(from, to);
      runs = runs_out;
      run_keys = out_keys;
    }
    const uint32_t blocks_per_row = (p.count + kBlockThreads - 1) / kBlockThreads;
    note_variant<EmitRunTag<kBytewise>>();
    hipLaunchKernelGGL((topk_emit_run<T, kBytewise>), dim3(p.rows * blocks_per_row), block, 0, s, in, values, indices,
                       from, a, run_keys, blocks_per_row);
    return hipGetLastError();
  }
  if (p.tiles == 1) {
    if (vector) {
      note_variant<TilesTag<true, false, true>>();
      hipLaunchKernelGGL((topk_tiles<T, true, false, true>), dim3(p.rows), block, 0, s, in, values, indices,
                         lists_a, a, 1u, tile_n, largest);
    } else {
      note_variant<TilesTag<false, kBytewise, true>>();
      hipLaunchKernelGGL((topk_tiles<T, false, kBytewise, true>), dim3(p.rows), block, 0, s, in, values,
                         indices, lists_a, a, 1u, tile_n, largest);
    }
    return hipGetLastError();
  }
  if (vector) {
    note_variant<TilesTag<true, false, false>>();
    hipLaunchKernelGGL((topk_tiles<T, true, false, false>), dim3(p.rows * p.tiles), block, 0, s, in, values,
                       indices, lists_a, a, p.tiles, kTile, largest);
  } else {
    note_variant<TilesTag<false, kBytewise, false>>();
    hipLaunchKernelGGL((topk_tiles<T, false, kBytewise, false>), dim3(p.rows * p.tiles), block, 0, s, in,
                       values, indices, lists_a, a, p.tiles, kTile, largest);
  }
  uint32_t lists = p.tiles;
  uint64_t *from = lists_a, *to = lists_b;
  while (lists > 1) {
    const uint32_t out = (lists + p.fan - 1) / p.fan;
    const uint32_t sort_n = pow2_at_least(std::min(lists, p.fan) * p.count, 64);
    if (out == 1) {
      note_variant<MergeTag<kBytewise, true>>();
      hipLaunchKernelGGL((topk_merge<T, kBytewise, true>), dim3(p.rows), block, 0, s, in, values, indices, from,
                         to, a, lists, p.fan, 1u, sort_n);
    } else {
      note_variant<MergeTag<kBytewise, false>>();
      hipLaunchKernelGGL((topk_merge<T, kBytewise, false>), dim3(p.rows * out), block, 0, s, in, values,
                         indices, from, to, a, lists, p.fan, out, sort_n);
    }
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
    // 8192-element tiles for long rows (32 elements per thread: the per-block work of finding the
    // bound is paid once per tile), 2048 otherwise; merges take as many
    // lists as 4096 keys hold (2048 when that already covers every tile of a row): 32 KiB of LDS.
    p->tile_elements = p->width > kTile ? kBlockThreads * 32 : kBlockThreads * 8;
    p->tiles = (p->width + p->tile_elements - 1) / p->tile_elements;
    p->fan = (p->tiles * p->count <= kBlockThreads * 8 ? kBlockThreads * 8 : kBlockThreads * 16) / p->count;
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
