// Concat: up to four plain inputs joined along one axis into a dense output, storage bits kept
// (src/compute_provider_cuda/concat_provider.cc:40-90: plain inputs, dense output, 1/2/4/8-byte
// elements, no overlap of inputs and output; the schema is src/compute_ops/operation.cc:1516-1564).
// Seen as [outer, extent, inner], input i is `outer` runs of extent_i * inner elements that land
// at element (o * total + offset_i) * inner of the output: a copy with two pitches.
#include <algorithm>

#include "device_common.h"
#include "kernels.h"

namespace hyle_hip {
namespace {

struct ConcatOperands {
  const unsigned char *base[4];
  uint64_t run_bytes[4];      // extent_i * inner * size
  uint64_t offset_bytes[4];   // offset_i * inner * size
  uint64_t out_pitch;         // total * inner * size
  uint32_t outer;
};

// Dense inputs: kUnit bytes per thread step (16 when every run, offset and pointer allows it,
// otherwise the element size).  grid.y is the input; a block takes up to kRunSteps * 256 units of
// one run, so the run and the place in it come from one division per block.
constexpr uint32_t kRunSteps = 4;
template <int kUnit>
__global__ __launch_bounds__(kBlockThreads) void concat_runs(ConcatOperands p, unsigned char *out) {
  const uint32_t input = blockIdx.y;
  const uint32_t units_per_run = (uint32_t)(p.run_bytes[input] / kUnit);
  if (units_per_run == 0) return;
  const uint32_t blocks_per_run = (units_per_run + kRunSteps * kBlockThreads - 1) / (kRunSteps * kBlockThreads);
  const uint32_t run = blockIdx.x / blocks_per_run, piece = blockIdx.x - run * blocks_per_run;
  if (run >= p.outer) return;
  const unsigned char *from = p.base[input] + (uint64_t)run * p.run_bytes[input];
  unsigned char *to = out + (uint64_t)run * p.out_pitch + p.offset_bytes[input];
#pragma unroll
  for (uint32_t j = 0; j < kRunSteps; ++j) {
    const uint32_t u = (piece * kRunSteps + j) * kBlockThreads + threadIdx.x;
    if (u >= units_per_run) break;
    if constexpr (kUnit == 16) store16_stream(to, u, load16_stream(from, u));
    else if constexpr (kUnit == 8) reinterpret_cast<uint64_t *>(to)[u] = reinterpret_cast<const uint64_t *>(from)[u];
    else if constexpr (kUnit == 4) reinterpret_cast<uint32_t *>(to)[u] = reinterpret_cast<const uint32_t *>(from)[u];
    else if constexpr (kUnit == 2) reinterpret_cast<uint16_t *>(to)[u] = reinterpret_cast<const uint16_t *>(from)[u];
    else to[u] = from[u];
  }
}

struct ConcatLayout {
  const unsigned char *base[4];
  uint32_t extent[4], offset[4];   // along the axis, in elements
  int64_t strides[4][kMaxRank];    // byte strides of each input
  uint32_t dims[kMaxRank];         // of the output; an input differs only on the axis
  int32_t rank, axis;
  uint32_t total;                  // the output's extent on the axis
};

// Any byte strides: one thread per element of input blockIdx.y, gathered bytewise.
template <int kSize>
__global__ __launch_bounds__(kBlockThreads) void concat_general(ConcatLayout p, unsigned char *out) {
  const uint32_t input = blockIdx.y;
  uint64_t elements = 1;
  for (int a = 0; a < p.rank; ++a) elements *= a == p.axis ? p.extent[input] : p.dims[a];
  const uint64_t step = (uint64_t)gridDim.x * kBlockThreads;
  for (uint64_t e = (uint64_t)blockIdx.x * kBlockThreads + threadIdx.x; e < elements; e += step) {
    uint64_t rest = e, to = 0, scale = 1;
    int64_t from = 0;
    for (int a = p.rank - 1; a >= 0; --a) {
      const uint32_t span = a == p.axis ? p.extent[input] : p.dims[a];
      const uint64_t c = rest % span;
      rest /= span;
      from += (int64_t)c * p.strides[input][a];
      to += (a == p.axis ? c + p.offset[input] : c) * scale;
      scale *= a == p.axis ? p.total : p.dims[a];
    }
    const unsigned char *source = p.base[input] + from;
#pragma unroll
    for (int b = 0; b < kSize; ++b) out[to * kSize + b] = source[b];
  }
}

uint32_t blocks_for(uint64_t units) {
  const uint64_t blocks = (units + kBlockThreads - 1) / kBlockThreads;
  return (uint32_t)(blocks < 1 ? 1 : (blocks > 16384 ? 16384 : blocks));
}

}  // namespace

// Launch-shape labels
template <int kUnit, bool kRuns> struct ConcatTag {
  static std::string text() { return std::string(kRuns ? "concat_runs/" : "concat_general/") + std::to_string(kUnit) + "-bytes"; }
};

hipError_t launch_concat(const ConcatParams &p, const void *const *inputs, void *out, hipStream_t stream) {
  if (p.elements == 0) return hipSuccess;
  unsigned char *o = static_cast<unsigned char *>(out);
  uint64_t most = 0;  // elements of the largest input
  for (uint32_t i = 0; i < p.inputs; ++i) most = std::max<uint64_t>(most, (uint64_t)p.outer * p.extent[i] * p.inner);
  if (most == 0) return hipSuccess;
  if (p.dense) {
    ConcatOperands c{};
    c.outer = p.outer;
    c.out_pitch = (uint64_t)p.total * p.inner * p.size;
    bool wide = (c.out_pitch | reinterpret_cast<uintptr_t>(out)) % 16 == 0;
    for (uint32_t i = 0; i < p.inputs; ++i) {
      c.base[i] = static_cast<const unsigned char *>(inputs[i]);
      c.run_bytes[i] = (uint64_t)p.extent[i] * p.inner * p.size;
      c.offset_bytes[i] = (uint64_t)p.offset[i] * p.inner * p.size;
      if (p.extent[i] != 0)
        wide = wide && (c.run_bytes[i] | c.offset_bytes[i] | reinterpret_cast<uintptr_t>(inputs[i])) % 16 == 0;
    }
    const int unit = wide ? 16 : p.size;
    uint64_t blocks = 1;  // of the input that needs most
    for (uint32_t i = 0; i < p.inputs; ++i) {
      const uint64_t units_per_run = c.run_bytes[i] / unit;
      blocks = std::max<uint64_t>(blocks, (units_per_run + kRunSteps * kBlockThreads - 1) / (kRunSteps * kBlockThreads) * p.outer);
    }
    const dim3 grid((uint32_t)blocks, p.inputs), block(kBlockThreads);
    switch (unit) {
      case 16: note_variant<ConcatTag<16, true>>(); hipLaunchKernelGGL((concat_runs<16>), grid, block, 0, stream, c, o); break;
      case 8: note_variant<ConcatTag<8, true>>(); hipLaunchKernelGGL((concat_runs<8>), grid, block, 0, stream, c, o); break;
      case 4: note_variant<ConcatTag<4, true>>(); hipLaunchKernelGGL((concat_runs<4>), grid, block, 0, stream, c, o); break;
      case 2: note_variant<ConcatTag<2, true>>(); hipLaunchKernelGGL((concat_runs<2>), grid, block, 0, stream, c, o); break;
      default: note_variant<ConcatTag<1, true>>(); hipLaunchKernelGGL((concat_runs<1>), grid, block, 0, stream, c, o); break;
    }
    return hipGetLastError();
  }
  ConcatLayout l{};
  l.rank = p.rank;
  l.axis = p.axis;
  l.total = p.total;
  for (int a = 0; a < kMaxRank; ++a) l.dims[a] = p.dims[a];
  for (uint32_t i = 0; i < p.inputs; ++i) {
    l.base[i] = static_cast<const unsigned char *>(inputs[i]);
    l.extent[i] = p.extent[i];
    l.offset[i] = p.offset[i];
    for (int a = 0; a < kMaxRank; ++a) l.strides[i][a] = p.strides[i][a];
  }
  const dim3 grid(blocks_for(most), p.inputs), block(kBlockThreads);
  switch (p.size) {
    case 8: note_variant<ConcatTag<8, false>>(); hipLaunchKernelGGL((concat_general<8>), grid, block, 0, stream, l, o); break;
    case 4: note_variant<ConcatTag<4, false>>(); hipLaunchKernelGGL((concat_general<4>), grid, block, 0, stream, l, o); break;
    case 2: note_variant<ConcatTag<2, false>>(); hipLaunchKernelGGL((concat_general<2>), grid, block, 0, stream, l, o); break;
    default: note_variant<ConcatTag<1, false>>(); hipLaunchKernelGGL((concat_general<1>), grid, block, 0, stream, l, o); break;
  }
  return hipGetLastError();
}

}  // namespace hyle_hip
