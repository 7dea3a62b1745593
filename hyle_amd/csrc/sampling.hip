// Sampling next to the vocabulary argmax (include/hyle/compute/sampling_ops.h:12-75).
//
// RandomBits: counter-addressed Philox4x32-10 words (third_party/random123_counter/philox.h:20-44),
// bit for bit the words every backend of the reference produces: word j of a row is lane j % 4 of
// the block whose counter is {j / 4 low, j / 4 high, draw low, draw high} under the row's key.
//
// Categorical: one draw per row of dense [rows, width] log-weights.  The reference lets each
// backend choose its draw algorithm (sampling_ops.h:50-55); this one follows the CPU provider's
// inverse CDF (src/compute_provider_native/sampling.cc:119-182) because it reads the row once at
// memory speed: one Philox block per row gives a 52-bit uniform u, the selected index is the
// first whose running mass exceeds u * total, masses being exp(x - max) summed in double.  The
// first dispatch leaves per tile of 4096 elements its maximum, its mass relative to that maximum
// and whether it holds NaN or +Inf; the second, one block per row, folds the tiles, finds the
// tile in which the running mass crosses the threshold and scans only that tile again.  A row
// with NaN, +Inf or no finite element writes nothing and sets the status word, which the host
// reports as InvalidArgument (sampling.cc:119-135,203-206).
#include "device_common.h"
#include "kernels.h"

namespace hyle_hip {
namespace {

struct PhiloxWords {
  uint32_t x0, x1, x2, x3;
};

__device__ __forceinline__ PhiloxWords philox_block(uint32_t key0, uint32_t key1, uint32_t draw0, uint32_t draw1,
                                                    uint64_t index) {
  PhiloxWords v{(uint32_t)index, (uint32_t)(index >> 32), draw0, draw1};
#pragma unroll
  for (int round = 0; round < 10; ++round) {
    // one 32 x 32 -> 64 product each (v_mad_u64_u32), not a high and a low multiply
    const uint64_t first = (uint64_t)0xD2511F53u * v.x0, second = (uint64_t)0xCD9E8D57u * v.x2;
    v = PhiloxWords{(uint32_t)(second >> 32) ^ v.x1 ^ key0, (uint32_t)second, (uint32_t)(first >> 32) ^ v.x3 ^ key1,
                    (uint32_t)first};
    key0 += 0x9E3779B9u;
    key1 += 0xBB67AE85u;
  }
  return v;
}

// One Philox block (four words) per thread over the flat block index: short or unaligned rows.
__global__ __launch_bounds__(kBlockThreads) void random_bits(const uint32_t *identities, uint32_t *out, uint32_t rows,
                                                             uint32_t word_count, uint32_t blocks_per_row, bool vector) {
  const uint64_t total = (uint64_t)rows * blocks_per_row;
  for (uint64_t i = (uint64_t)blockIdx.x * kBlockThreads + threadIdx.x; i < total; i += (uint64_t)gridDim.x * kBlockThreads) {
    const uint32_t row = (uint32_t)(i / blocks_per_row), column = (uint32_t)(i - (uint64_t)row * blocks_per_row);
    const uint32_t *identity = identities + (size_t)row * 4;  // element-aligned, as the reference asks
    const PhiloxWords w = philox_block(identity[0], identity[1], identity[2], identity[3], column);
    uint32_t *to = out + (uint64_t)row * word_count + (uint64_t)column * 4;
    if (vector) {
      store16_stream(to, 0, u32x4{w.x0, w.x1, w.x2, w.x3});
    } else {
      const uint32_t words[4] = {w.x0, w.x1, w.x2, w.x3};
      const uint32_t left = word_count - column * 4;
#pragma unroll
      for (uint32_t lane = 0; lane < 4; ++lane)
        if (lane < left) to[lane] = words[lane];
    }
  }
}

// Long rows: the row is the block's (its identity sits in scalar registers and nothing is
// divided), a thread makes four blocks 256 apart, so every store of a wave is 1 KiB in one piece
// and a thread's earlier stores drain while it works on the next block.
constexpr int kBitsPerThread = 4;
__global__ __launch_bounds__(kBlockThreads) void random_bits_rows(const uint32_t *identities, uint32_t *out, uint32_t rows,
                                                                  uint32_t word_count, uint32_t blocks_per_row) {
  for (uint32_t row = blockIdx.y; row < rows; row += gridDim.y) {
    const uint32_t *identity = identities + (size_t)row * 4;
    const uint32_t key0 = identity[0], key1 = identity[1], draw0 = identity[2], draw1 = identity[3];
    uint32_t *to = out + (uint64_t)row * word_count;
#pragma unroll
    for (int j = 0; j < kBitsPerThread; ++j) {
      const uint32_t column = (blockIdx.x * kBitsPerThread + j) * kBlockThreads + threadIdx.x;
      if (column < blocks_per_row) {
        const PhiloxWords w = philox_block(key0, key1, draw0, draw1, column);
        store16_stream(to, column, u32x4{w.x0, w.x1, w.x2, w.x3});
      }
    }
  }
}

// ---- Categorical ------------------------------------------------------------------------------
constexpr int kPerThread = kCategoricalTile / kBlockThreads;  // 16

// exp(t) for t <= 0 (0 for -inf): t * log2(e) as a rounded product plus its exact residual, so
// the hardware exp2 sees an argument good to about 2e-8 * |t|.
__device__ __forceinline__ float exp_nonpositive(float t) {
  constexpr float kLog2e = 1.44269504088896340736f;
  constexpr float kLn2 = 0.69314718055994530942f;
  t = fmaxf(t, -200.0f);
  const float hi = t * kLog2e;
  const float lo = __builtin_fmaf(t, kLog2e, -hi);
  const float p = __builtin_amdgcn_exp2f(hi);
  return __builtin_fmaf(p, lo * kLn2, p);
}

__device__ __forceinline__ bool invalid_weight(float v) {
  return __builtin_amdgcn_class(v, 0x001 | 0x002 | 0x200);  // sNaN | qNaN | +inf
}

// The 16 elements of a thread in a tile: with whole 16-byte vectors, vector j of the thread holds
// elements (j * 256 + thread) * kVec ...; element by element, step j is element j * 256 + thread.
// Places past the row read as -inf (no mass).  `place(j, e)` is the element's index in the tile.
template <class T, bool kVector> struct TileValues {
  static constexpr int kVec = kVector ? Traits<T>::kVec : 1;
  static constexpr int kSteps = kPerThread / kVec;
  float v[kPerThread];
  static __device__ __forceinline__ uint32_t place(int j, int e) { return (uint32_t)(j * kBlockThreads + threadIdx.x) * kVec + e; }
  __device__ __forceinline__ void load(const void *row, uint32_t first, uint32_t count) {
    constexpr float kNone = -__builtin_huge_valf();
    if constexpr (kVector) {
#pragma unroll
      for (int j = 0; j < kSteps; ++j) {
        const uint32_t at = place(j, 0);  // count is a multiple of kVec on this route
        float part[kVec];
        if (at < count) {
          Traits<T>::unpack(load16_stream(static_cast<const unsigned char *>(row) + (size_t)first * Traits<T>::kSize, at / kVec), part);
        } else {
#pragma unroll
          for (int e = 0; e < kVec; ++e) part[e] = kNone;
        }
#pragma unroll
        for (int e = 0; e < kVec; ++e) v[j * kVec + e] = part[e];
      }
    } else {
#pragma unroll
      for (int j = 0; j < kSteps; ++j) v[j] = place(j, 0) < count ? Traits<T>::load(row, (size_t)first + place(j, 0)) : kNone;
    }
  }
};

__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
  for (int step = 1; step < kWaveLanes; step *= 2) v += __shfl_xor(v, step, kWaveLanes);
  return v;
}

template <class T, bool kVector>
__global__ __launch_bounds__(kBlockThreads) void categorical_tiles(const void *logits, uint32_t width, uint32_t tiles,
                                                                   CategoricalTile *out, uint32_t *status) {
  __shared__ float joint[kBlockThreads / kWaveLanes];
  __shared__ double masses[kBlockThreads / kWaveLanes];
  if (blockIdx.x == 0 && threadIdx.x == 0) *status = 0;  // the rows' dispatch sets it
  const uint32_t row = blockIdx.x / tiles, tile = blockIdx.x - row * tiles;
  const uint32_t first = tile * kCategoricalTile;
  const uint32_t count = width - first < (uint32_t)kCategoricalTile ? width - first : (uint32_t)kCategoricalTile;
  const void *base = static_cast<const unsigned char *>(logits) + (size_t)row * width * Traits<T>::kSize;
  TileValues<T, kVector> values;
  values.load(base, first, count);
  bool invalid = false;
  float maximum = -__builtin_huge_valf();
#pragma unroll
  for (int i = 0; i < kPerThread; ++i) {
    invalid = invalid || invalid_weight(values.v[i]);
    maximum = fmaxf(maximum, values.v[i]);  // ignores NaN; the flag carries it
  }
  maximum = row_max<kBlockThreads>(maximum, joint);
  double mass = 0;
  if (maximum > -__builtin_huge_valf()) {
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) mass += (double)exp_nonpositive(values.v[i] - maximum);
  }
  mass = wave_sum(mass);
  if ((threadIdx.x & (kWaveLanes - 1)) == 0) masses[threadIdx.x / kWaveLanes] = mass;
  const int any_invalid = __syncthreads_or(invalid ? 1 : 0);
  if (threadIdx.x == 0) {
    double total = 0;
#pragma unroll
    for (int w = 0; w < kBlockThreads / kWaveLanes; ++w) total += masses[w];
    out[blockIdx.x] = CategoricalTile{maximum, any_invalid ? 1u : 0u, total};
  }
}

// Scan of one double per thread over the block, in thread order: returns the sum of the threads
// below (exactly the inclusive value the thread below holds) and leaves the inclusive value and
// the block's total in `through` and `total`.  Two barriers.
__device__ __forceinline__ double block_scan(double v, double *wave_totals, double *through, double *total) {
  const int lane = threadIdx.x & (kWaveLanes - 1), wave = threadIdx.x / kWaveLanes;
#pragma unroll
  for (int step = 1; step < kWaveLanes; step *= 2) {
    const double below = __shfl_up(v, step, kWaveLanes);
    if (lane >= step) v += below;
  }
  const double previous = __shfl_up(v, 1, kWaveLanes);
  if (lane == kWaveLanes - 1) wave_totals[wave] = v;
  __syncthreads();
  double before = 0, all = 0;
#pragma unroll
  for (int w = 0; w < kBlockThreads / kWaveLanes; ++w) {
    if (w < wave) before += wave_totals[w];
    all += wave_totals[w];
  }
  __syncthreads();
  *total = all;
  *through = v + before;
  return lane == 0 ? before : previous + before;
}

// The 16 consecutive elements of a thread in a tile (thread t holds elements 16 t ... 16 t + 15), so
// that one scan over the threads orders the whole tile.  Places past the row read as -inf.
template <class T, bool kVector>
__device__ __forceinline__ void load_consecutive(const void *row, uint32_t first, uint32_t count, float (&v)[kPerThread]) {
  constexpr float kNone = -__builtin_huge_valf();
  const uint32_t mine = threadIdx.x * kPerThread;
  if constexpr (kVector) {
    constexpr int kVec = Traits<T>::kVec;
    const unsigned char *base = static_cast<const unsigned char *>(row) + ((size_t)first + mine) * Traits<T>::kSize;
#pragma unroll
    for (int j = 0; j < kPerThread / kVec; ++j) {
      float part[kVec];
      if (mine + j * kVec < count) {  // count is a multiple of kVec on this route
        Traits<T>::unpack(load16(base, j), part);
      } else {
#pragma unroll
        for (int e = 0; e < kVec; ++e) part[e] = kNone;
      }
#pragma unroll
      for (int e = 0; e < kVec; ++e) v[j * kVec + e] = part[e];
    }
  } else {
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) v[i] = mine + i < count ? Traits<T>::load(row, (size_t)first + mine + i) : kNone;
  }
}

// What the thread that holds the crossing tile tells the block.
struct Crossing {
  double residual;   // the threshold less the mass before the tile, on the row's scale
  uint32_t tile;     // 0xFFFFFFFF: rounding left the threshold at the row's total
  float tile_maximum, scale;  // scale = exp(tile_maximum - row maximum)
};

template <class T, bool kVector, bool kScored>
__global__ __launch_bounds__(kBlockThreads) void categorical_rows(const void *logits, const uint32_t *identities,
                                                                  uint32_t width, uint32_t tiles, const CategoricalTile *parts,
                                                                  int32_t *indices, float *scores, uint32_t *status) {
  __shared__ float joint[kBlockThreads / kWaveLanes];
  __shared__ double wave_totals[kBlockThreads / kWaveLanes];
  __shared__ Crossing crossing;
  __shared__ uint32_t found, claim;
  constexpr float kInfinity = __builtin_huge_valf();
  const uint32_t row = blockIdx.x;
  const CategoricalTile *mine = parts + (size_t)row * tiles;
  const void *base = static_cast<const unsigned char *>(logits) + (size_t)row * width * Traits<T>::kSize;
  const uint32_t *identity = identities + (size_t)row * 4;
  const uint32_t key0 = identity[0], key1 = identity[1], draw0 = identity[2], draw1 = identity[3];
  // the row's maximum; a tile with NaN or +inf counts as +inf, which no valid tile reaches
  float maximum = -kInfinity;
  for (uint32_t t = threadIdx.x; t < tiles; t += kBlockThreads) maximum = fmaxf(maximum, mine[t].invalid ? kInfinity : mine[t].maximum);
  maximum = row_max<kBlockThreads>(maximum, joint);
  if (!(maximum > -kInfinity && maximum < kInfinity)) {
    if (threadIdx.x == 0) *status = kStatusInvalidNumericInput;
    return;
  }
  // masses on the row's scale, summed in tile order: a thread owns a run of consecutive tiles
  const uint32_t per_thread = (tiles + kBlockThreads - 1) / kBlockThreads;
  const uint32_t begin = threadIdx.x * per_thread < tiles ? threadIdx.x * per_thread : tiles;
  const uint32_t end = begin + per_thread < tiles ? begin + per_thread : tiles;
  auto scale_of = [&](uint32_t t) { return exp_nonpositive(mine[t].maximum - maximum); };  // 0 for a tile without mass
  double own = 0;
  for (uint32_t t = begin; t < end; ++t) own += mine[t].mass * (double)scale_of(t);
  double total = 0, through = 0;
  const double before = block_scan(own, wave_totals, &through, &total);
  const PhiloxWords draw = philox_block(key0, key1, draw0, draw1, 0);
  // the 52-bit midpoint is exact in double at both ends (sampling.cc:155-158)
  const double uniform = ((double)draw.x0 * 0x1p20 + (double)(draw.x1 >> 12) + 0.5) * 0x1p-52;
  const double threshold = total * uniform;
  if (threadIdx.x == 0) {
    crossing.tile = 0xFFFFFFFFu;
    claim = 0xFFFFFFFFu;
  }
  __syncthreads();
  // The scan's running sums are associated differently from lane to lane, so they need not be
  // monotone in their last bit: a thread without mass may see the threshold between its equal
  // `before` and `through`, and two neighbours may both see it.  Only threads with mass of their
  // own may hold the crossing, and the lowest of them answers.
  const bool candidate = own > 0 && !(before > threshold) && through > threshold;
  if (candidate) atomicMin(&claim, threadIdx.x);
  __syncthreads();
  if (candidate && claim == threadIdx.x) {  // the first tile whose running mass exceeds the threshold is here
    double running = before;
    uint32_t tile = 0xFFFFFFFFu, last_with_mass = 0xFFFFFFFFu;
    for (uint32_t t = begin; t < end; ++t) {
      const double share = mine[t].mass * (double)scale_of(t);
      if (share > 0) last_with_mass = t;
      if (running + share > threshold) {
        tile = t;
        break;
      }
      running += share;
    }
    if (tile == 0xFFFFFFFFu) {  // the scan's sum and this walk's differ in their last bit: the run's last mass
      tile = last_with_mass;
      running = threshold;
    }
    // (a run without mass cannot get here; if it did, the crossing stays unset and the row's last
    // maximum answers below, never an index outside the tiles)
    if (tile != 0xFFFFFFFFu) crossing = Crossing{threshold - running, tile, mine[tile].maximum, scale_of(tile)};
  }
  __syncthreads();
  if (crossing.tile == 0xFFFFFFFFu) {
    // rounding left the threshold at the total: the last element equal to the maximum (sampling.cc:168-173)
    if (threadIdx.x == 0) found = 0;
    __syncthreads();
    uint32_t last = 0;
    for (uint32_t c = threadIdx.x; c < width; c += kBlockThreads)
      if (Traits<T>::load(base, c) == maximum) last = c;
    atomicMax(&found, last);
    __syncthreads();
    if (threadIdx.x == 0) {
      indices[row] = (int32_t)found;
      if constexpr (kScored) scores[row] = -logf((float)total);
    }
    return;
  }
  const uint32_t first = crossing.tile * kCategoricalTile;
  const uint32_t count = width - first < (uint32_t)kCategoricalTile ? width - first : (uint32_t)kCategoricalTile;
  float v[kPerThread];
  load_consecutive<T, kVector>(base, first, count, v);
  // the residual on the tile's own scale, the one its mass was summed on
  const double residual = crossing.residual / (double)crossing.scale;
  float weights[kPerThread];
  double mass = 0;
#pragma unroll
  for (int i = 0; i < kPerThread; ++i) {
    weights[i] = exp_nonpositive(v[i] - crossing.tile_maximum);
    mass += (double)weights[i];
  }
  double tile_total = 0, mass_through = 0;
  const double mass_before = block_scan(mass, wave_totals, &mass_through, &tile_total);
  // exactly one thread holds the crossing; none when rounding left the residual at the tile's total,
  // and then the thread with the tile's last mass answers
  const bool last_mass = !(tile_total > residual) && mass > 0 && mass_through == tile_total;
  if ((!(mass_before > residual) && mass_through > residual) || last_mass) {
    double running = mass_before;
    int selected = -1, last_positive = -1;
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) {
      running += (double)weights[i];
      if (weights[i] > 0) last_positive = i;
      if (selected < 0 && running > residual) selected = i;
    }
    if (selected < 0) selected = last_positive;
    float chosen = v[0];
#pragma unroll
    for (int i = 1; i < kPerThread; ++i) chosen = selected == i ? v[i] : chosen;
    indices[row] = (int32_t)(first + threadIdx.x * kPerThread + selected);
    if constexpr (kScored) {
      // (x - max) - log(total): the logarithm in f32 with the rounding of the total put back
      const float total32 = (float)total;
      const double log_total = (double)logf(total32) + (total - (double)total32) / (double)total32;
      scores[row] = (float)((double)chosen - (double)maximum - log_total);
    }
  }
}

// Launch-shape labels
template <bool kVector> struct CategoricalTilesTag {
  static std::string text() { return std::string("categorical_tiles/") + (kVector ? "vector" : "scalar"); }
};
template <bool kVector, bool kScored> struct CategoricalRowsTag {
  static std::string text() { return std::string("categorical_rows/") + (kVector ? "vector" : "scalar") + (kScored ? "/scored" : ""); }
};
template <int kForm> struct RandomBitsTag {  // 0 rows of blocks, 1 flat
  static std::string text() { return kForm == 0 ? "random_bits_rows" : "random_bits"; }
};

template <class T, bool kVector>
hipError_t run_categorical(const CategoricalParams &p, const void *logits, const uint32_t *identities, int32_t *indices,
                           float *scores, void *workspace, hipStream_t stream) {
  CategoricalTile *parts = static_cast<CategoricalTile *>(workspace);
  uint32_t *status = reinterpret_cast<uint32_t *>(static_cast<unsigned char *>(workspace) + p.status_offset);
  const dim3 block(kBlockThreads);
  note_variant<CategoricalTilesTag<kVector>>();
  hipLaunchKernelGGL((categorical_tiles<T, kVector>), dim3(p.rows * p.tiles), block, 0, stream, logits, p.width, p.tiles, parts,
                     status);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return err;
  if (p.scored) {
    note_variant<CategoricalRowsTag<kVector, true>>();
    hipLaunchKernelGGL((categorical_rows<T, kVector, true>), dim3(p.rows), block, 0, stream, logits, identities, p.width,
                       p.tiles, parts, indices, scores, status);
  } else {
    note_variant<CategoricalRowsTag<kVector, false>>();
    hipLaunchKernelGGL((categorical_rows<T, kVector, false>), dim3(p.rows), block, 0, stream, logits, identities, p.width,
                       p.tiles, parts, indices, scores, status);
  }
  return hipGetLastError();
}

template <class T>
hipError_t run_categorical_typed(const CategoricalParams &p, const void *logits, const uint32_t *identities, int32_t *indices,
                                 float *scores, void *workspace, bool vector_aligned, hipStream_t stream) {
  // whole 16-byte vectors: every row starts on one and holds a whole number of them
  const bool vector = vector_aligned && ((uint64_t)p.width * Traits<T>::kSize) % 16 == 0;
  if (vector) return run_categorical<T, true>(p, logits, identities, indices, scores, workspace, stream);
  return run_categorical<T, false>(p, logits, identities, indices, scores, workspace, stream);
}

}  // namespace

hipError_t launch_random_bits(const RandomBitsParams &p, const void *identities, void *out, hipStream_t stream) {
  if (p.rows == 0 || p.word_count == 0) return hipSuccess;
  const uint32_t blocks_per_row = (p.word_count + 3) / 4;
  const uint64_t total = (uint64_t)p.rows * blocks_per_row;
  uint64_t blocks = (total + kBlockThreads - 1) / kBlockThreads;
  blocks = blocks > 65535 ? 65535 : blocks;
  const bool vector = p.word_count % 4 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
  if (vector && blocks_per_row >= kBlockThreads) {
    const uint32_t per_block = kBlockThreads * kBitsPerThread;
    const dim3 grid((blocks_per_row + per_block - 1) / per_block, p.rows < 65535u ? p.rows : 65535u);
    note_variant<RandomBitsTag<0>>();
    hipLaunchKernelGGL(random_bits_rows, grid, dim3(kBlockThreads), 0, stream, static_cast<const uint32_t *>(identities),
                       static_cast<uint32_t *>(out), p.rows, p.word_count, blocks_per_row);
    return hipGetLastError();
  }
  note_variant<RandomBitsTag<1>>();
  hipLaunchKernelGGL(random_bits, dim3((uint32_t)blocks), dim3(kBlockThreads), 0, stream, static_cast<const uint32_t *>(identities),
                     static_cast<uint32_t *>(out), p.rows, p.word_count, blocks_per_row, vector);
  return hipGetLastError();
}

hipError_t launch_categorical(Elem type, const CategoricalParams &p, const void *logits, const void *identities, void *indices,
                              void *scores, void *workspace, bool vector_aligned, hipStream_t stream) {
  if (p.rows == 0) return hipSuccess;
  const uint32_t *ids = static_cast<const uint32_t *>(identities);
  int32_t *out = static_cast<int32_t *>(indices);
  float *score = static_cast<float *>(scores);
  switch (type) {
    case Elem::kF32: return run_categorical_typed<F32>(p, logits, ids, out, score, workspace, vector_aligned, stream);
    case Elem::kF16: return run_categorical_typed<F16>(p, logits, ids, out, score, workspace, vector_aligned, stream);
    case Elem::kBF16: return run_categorical_typed<BF16>(p, logits, ids, out, score, workspace, vector_aligned, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace hyle_hip
