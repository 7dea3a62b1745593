// argmax.hip -- TopK(count = 1, largest) over the last axis for gfx950: the
// greedy-token argmax over vocabulary logits.
//
// A few very wide rows cannot fill 256 CUs with one block per row, so each row is
// cut into tiles; every block scans one tile with 128-bit loads and leaves its
// best (value, index) candidate in the workspace, then one block per row folds
// the candidates.  Ordering is the reference's TopK rule
// (src/compute_provider_cuda/collectives.cu:478-495): a number beats NaN, a
// larger number beats a smaller one, ties (including -0 against +0 and NaN
// against NaN) go to the lower index.  The value output carries the original
// storage bits of the winner.
#include "device_common.h"
#include "kernels.h"

namespace hyle_hip {
namespace {

struct Candidate {
  float value;
  int32_t index;
};

__device__ __forceinline__ LaneArg block_best(LaneArg best, LaneArg *joint) {
  best = group_reduce<kWaveLanes>(best, [](LaneArg a, LaneArg b) { return arg_best(a, b); });
  if ((threadIdx.x & (kWaveLanes - 1)) == 0) joint[threadIdx.x / kWaveLanes] = best;
  __syncthreads();
  return arg_best(arg_best(joint[0], joint[1]), arg_best(joint[2], joint[3]));
}

// A lane walks its elements in increasing index order, so "strictly better"
// keeps the lowest index among equals.
__device__ __forceinline__ void consider(LaneArg &best, float value, int32_t index) {
  const bool best_nan = best.value != best.value;
  const bool better = best.index < 0 || (best_nan && value == value) || value > best.value;
  if (better) best = LaneArg{value, index};
}

template <class T, bool kVector>
__global__ __launch_bounds__(kBlockThreads) void argmax_tiles(const void *x, Candidate *partial,
                                                              uint32_t width, uint32_t tiles,
                                                              uint32_t tile_elems) {
  constexpr int kVec = Traits<T>::kVec;
  __shared__ LaneArg joint[4];
  const uint32_t row = blockIdx.x / tiles, tile = blockIdx.x % tiles;
  const uint32_t begin = tile * tile_elems;
  const uint32_t end = begin + tile_elems < width ? begin + tile_elems : width;
  LaneArg best{0.0f, -1};
  if constexpr (kVector) {
    // width % kVec == 0 and tile_elems % kVec == 0: whole vectors only
    const size_t row_vec = (size_t)row * (width / kVec);
    const uint32_t vec_end = end / kVec;
    uint32_t vec = begin / kVec + threadIdx.x;
    // two vectors in flight per lane
    for (; vec + kBlockThreads < vec_end; vec += 2 * kBlockThreads) {
      float a[kVec], b[kVec];
      Traits<T>::unpack(load16_stream(x, row_vec + vec), a);
      Traits<T>::unpack(load16_stream(x, row_vec + vec + kBlockThreads), b);
#pragma unroll
      for (int j = 0; j < kVec; ++j) consider(best, a[j], (int32_t)(vec * kVec + j));
#pragma unroll
      for (int j = 0; j < kVec; ++j)
        consider(best, b[j], (int32_t)((vec + kBlockThreads) * kVec + j));
    }
    if (vec < vec_end) {
      float a[kVec];
      Traits<T>::unpack(load16_stream(x, row_vec + vec), a);
#pragma unroll
      for (int j = 0; j < kVec; ++j) consider(best, a[j], (int32_t)(vec * kVec + j));
    }
  } else {
    const size_t base = (size_t)row * width;
    for (uint32_t i = begin + threadIdx.x; i < end; i += kBlockThreads)
      consider(best, Traits<T>::load(x, base + i), (int32_t)i);
  }
  best = block_best(best, joint);
  if (threadIdx.x == 0) partial[blockIdx.x] = Candidate{best.value, best.index};
}

template <class T>
__global__ __launch_bounds__(kBlockThreads) void argmax_finish(const void *x,
                                                               const Candidate *partial, void *values,
                                                               int32_t *indices, uint32_t width,
                                                               uint32_t tiles) {
  __shared__ LaneArg joint[4];
  const uint32_t row = blockIdx.x;
  LaneArg best{0.0f, -1};
  for (uint32_t t = threadIdx.x; t < tiles; t += kBlockThreads) {
    const Candidate c = partial[(size_t)row * tiles + t];
    best = arg_best(best, LaneArg{c.value, c.index});
  }
  best = block_best(best, joint);
  if (threadIdx.x == 0) {
    indices[row] = best.index;
    if (values != nullptr) {
      // copy the winner's storage bits untouched
      const size_t at = (size_t)row * width + (uint32_t)best.index;
      if constexpr (Traits<T>::kSize == 4)
        static_cast<uint32_t *>(values)[row] = static_cast<const uint32_t *>(x)[at];
      else
        static_cast<uint16_t *>(values)[row] = static_cast<const uint16_t *>(x)[at];
    }
  }
}

template <class T>
hipError_t run(const ArgmaxParams &p, const void *x, void *values, int32_t *indices, void *workspace,
               bool vectorised, hipStream_t s) {
  const uint32_t rows = (uint32_t)p.shape.rows, width = p.shape.width;
  auto *partial = static_cast<Candidate *>(workspace);
  const bool vec = vectorised && width % Traits<T>::kVec == 0;
  if (vec)
    hipLaunchKernelGGL((argmax_tiles<T, true>), dim3(rows * p.tiles), dim3(kBlockThreads), 0, s, x,
                       partial, width, p.tiles, p.tile_elems);
  else
    hipLaunchKernelGGL((argmax_tiles<T, false>), dim3(rows * p.tiles), dim3(kBlockThreads), 0, s, x,
                       partial, width, p.tiles, p.tile_elems);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return err;
  hipLaunchKernelGGL((argmax_finish<T>), dim3(rows), dim3(kBlockThreads), 0, s, x, partial, values,
                     indices, width, p.tiles);
  return hipGetLastError();
}

}  // namespace

// Tiles are multiples of 1024 elements (whole vectors for every storage type).
// Aim for a few blocks per CU so the scan is spread over the whole chip, but keep
// at least 4096 elements per tile so a block has enough loads in flight.
void argmax_plan(uint64_t rows, uint32_t width, int compute_units, ArgmaxParams *p) {
  p->shape.rows = rows;
  p->shape.width = width;
  const uint64_t want_blocks = (uint64_t)(compute_units > 0 ? compute_units : 256) * 8;
  uint64_t tiles = rows == 0 ? 1 : (want_blocks + rows - 1) / rows;
  if (tiles < 1) tiles = 1;
  uint64_t tile_elems = (width + tiles - 1) / tiles;
  if (tile_elems < 4096) tile_elems = 4096;
  tile_elems = (tile_elems + 1023) / 1024 * 1024;
  p->tile_elems = (uint32_t)tile_elems;
  p->tiles = width == 0 ? 1 : (uint32_t)((width + tile_elems - 1) / tile_elems);
}

size_t argmax_workspace_bytes(const ArgmaxParams &p) {
  return (size_t)p.shape.rows * p.tiles * sizeof(Candidate);
}

hipError_t launch_argmax(Elem type, const ArgmaxParams &p, const void *x, void *values,
                         int32_t *indices, void *workspace, bool vectorised, hipStream_t stream) {
  if (p.shape.rows == 0 || p.shape.width == 0) return hipSuccess;
  switch (type) {
    case Elem::kF32: return run<F32>(p, x, values, indices, workspace, vectorised, stream);
    case Elem::kF16: return run<F16>(p, x, values, indices, workspace, vectorised, stream);
    case Elem::kBF16: return run<BF16>(p, x, values, indices, workspace, vectorised, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace hyle_hip
