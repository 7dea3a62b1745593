// device_common.h -- device-side building blocks shared by the gfx950 kernels:
// storage codecs, 128-bit vector access and wave64 reductions.
//
// Storage codecs follow include/hyle/simd/dtype.h:55-121 of the reference:
// bf16 is RN-even with NaN keeping its upper payload and gaining the quiet bit;
// f16 uses the hardware converters (IEEE RN-even, exact subnormals) with NaN
// forced to mantissa 0x3FF.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hyle_hip {

constexpr int kBlockThreads = 256;
constexpr int kWaveLanes = 64;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

struct F32 {};
struct F16 {};
struct BF16 {};

__device__ __forceinline__ float bits_f32(uint32_t u) { return __uint_as_float(u); }
__device__ __forceinline__ uint32_t f32_bits(float f) { return __float_as_uint(f); }

// f32 -> bf16 with the gfx950 converter (v_cvt_pk_bf16_f32).  It was compared on the
// device with the reference rule of include/hyle/simd/dtype.h:114-121 (RN-even, NaN keeps
// its upper payload and gains the quiet bit) over all 2^32 f32 patterns: identical.
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const f32x2 in = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(in, bf16x2));
}
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  return (uint16_t)(pack_bf16x2(f, 0.0f) & 0xFFFFu);
}
// the value after one trip through bf16 storage
__device__ __forceinline__ float bf16_round_trip(float f) {
  return bits_f32(pack_bf16x2(f, 0.0f) << 16);
}
__device__ __forceinline__ float bf16_lo(uint32_t w) { return bits_f32(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return bits_f32(w & 0xFFFF0000u); }

__device__ __forceinline__ float f16_to_f32(uint16_t h) {
  return (float)__builtin_bit_cast(_Float16, h);
}
// The value is made opaque before it is narrowed: left alone, the compiler fuses a preceding
// multiply by a widened f16 into v_fma_mixlo_f16 (a * b + 0), and that +0 addend turns a
// product of -0 into +0.
__device__ __forceinline__ uint16_t f32_to_f16(float f) {
  asm("" : "+v"(f));
  const uint16_t h = __builtin_bit_cast(uint16_t, (_Float16)f);
  const uint16_t nan = (uint16_t)(((f32_bits(f) >> 16) & 0x8000u) | 0x7FFFu);
  return (f != f) ? nan : h;
}

// Two values narrowed by one v_cvt_pk_f16_f32, under the same rules as f32_to_f16.
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi) {
  asm("" : "+v"(lo), "+v"(hi));
  const f32x2 in = {lo, hi};
  const uint32_t pair = __builtin_bit_cast(uint32_t, __builtin_convertvector(in, f16x2));
  const uint32_t nans = ((f32_bits(lo) >> 16) & 0x8000u) | (f32_bits(hi) & 0x80000000u) | 0x7FFF7FFFu;
  const uint32_t take = (lo != lo ? 0x0000FFFFu : 0u) | (hi != hi ? 0xFFFF0000u : 0u);
  return (pair & ~take) | (nans & take);
}

// ---- per-type traits: element size, elements per 16-byte vector, scalar and
// ---- vector load/store through f32 -----------------------------------------
template <class T> struct Traits;

template <> struct Traits<F32> {
  static constexpr int kSize = 4;
  static constexpr int kVec = 4;
  static __device__ __forceinline__ float load(const void *p, size_t i) {
    return static_cast<const float *>(p)[i];
  }
  static __device__ __forceinline__ void store(void *p, size_t i, float v) {
    static_cast<float *>(p)[i] = v;
  }
  static __device__ __forceinline__ float round(float v) { return v; }
  static __device__ __forceinline__ void unpack(u32x4 w, float (&v)[4]) {
    v[0] = bits_f32(w.x); v[1] = bits_f32(w.y); v[2] = bits_f32(w.z); v[3] = bits_f32(w.w);
  }
  static __device__ __forceinline__ u32x4 pack(const float (&v)[4]) {
    u32x4 w;
    w.x = f32_bits(v[0]); w.y = f32_bits(v[1]); w.z = f32_bits(v[2]); w.w = f32_bits(v[3]);
    return w;
  }
};

template <> struct Traits<BF16> {
  static constexpr int kSize = 2;
  static constexpr int kVec = 8;
  static __device__ __forceinline__ float load(const void *p, size_t i) {
    return bits_f32((uint32_t)static_cast<const uint16_t *>(p)[i] << 16);
  }
  static __device__ __forceinline__ void store(void *p, size_t i, float v) {
    static_cast<uint16_t *>(p)[i] = f32_to_bf16(v);
  }
  // value after one trip through storage
  static __device__ __forceinline__ float round(float v) { return bf16_round_trip(v); }
  static __device__ __forceinline__ void unpack(u32x4 w, float (&v)[8]) {
    v[0] = bf16_lo(w.x); v[1] = bf16_hi(w.x); v[2] = bf16_lo(w.y); v[3] = bf16_hi(w.y);
    v[4] = bf16_lo(w.z); v[5] = bf16_hi(w.z); v[6] = bf16_lo(w.w); v[7] = bf16_hi(w.w);
  }
  static __device__ __forceinline__ u32x4 pack(const float (&v)[8]) {
    u32x4 w;
    w.x = pack_bf16x2(v[0], v[1]); w.y = pack_bf16x2(v[2], v[3]);
    w.z = pack_bf16x2(v[4], v[5]); w.w = pack_bf16x2(v[6], v[7]);
    return w;
  }
};

template <> struct Traits<F16> {
  static constexpr int kSize = 2;
  static constexpr int kVec = 8;
  static __device__ __forceinline__ float load(const void *p, size_t i) {
    return f16_to_f32(static_cast<const uint16_t *>(p)[i]);
  }
  static __device__ __forceinline__ void store(void *p, size_t i, float v) {
    static_cast<uint16_t *>(p)[i] = f32_to_f16(v);
  }
  static __device__ __forceinline__ float round(float v) { return f16_to_f32(f32_to_f16(v)); }
  static __device__ __forceinline__ void unpack(u32x4 w, float (&v)[8]) {
    v[0] = f16_to_f32((uint16_t)w.x); v[1] = f16_to_f32((uint16_t)(w.x >> 16));
    v[2] = f16_to_f32((uint16_t)w.y); v[3] = f16_to_f32((uint16_t)(w.y >> 16));
    v[4] = f16_to_f32((uint16_t)w.z); v[5] = f16_to_f32((uint16_t)(w.z >> 16));
    v[6] = f16_to_f32((uint16_t)w.w); v[7] = f16_to_f32((uint16_t)(w.w >> 16));
  }
  static __device__ __forceinline__ u32x4 pack(const float (&v)[8]) {
    u32x4 w;
    w.x = pack_f16x2(v[0], v[1]); w.y = pack_f16x2(v[2], v[3]);
    w.z = pack_f16x2(v[4], v[5]); w.w = pack_f16x2(v[6], v[7]);
    return w;
  }
};

// A fence for the compiler only: the loads written before it are issued before it and no
// later load is hoisted above it, and the named registers must hold their loaded values here.
// Used after a group of independent loads so that they are all in flight together instead of
// being sunk next to their first use, one memory latency after another.
__device__ __forceinline__ void loads_issued(u32x4 &a) { asm volatile("" : "+v"(a) : : "memory"); }
__device__ __forceinline__ void loads_issued(uint32_t &a) { asm volatile("" : "+v"(a) : : "memory"); }

// 16-byte global access.  Streaming data is touched once, so loads and stores
// carry the non-temporal hint; small reused operands use the plain forms.
__device__ __forceinline__ u32x4 load16_stream(const void *base, size_t vec) {
  return __builtin_nontemporal_load(static_cast<const u32x4 *>(base) + vec);
}
__device__ __forceinline__ u32x4 load16(const void *base, size_t vec) {
  return static_cast<const u32x4 *>(base)[vec];
}
__device__ __forceinline__ void store16_stream(void *base, size_t vec, u32x4 w) {
  __builtin_nontemporal_store(w, static_cast<u32x4 *>(base) + vec);
}
__device__ __forceinline__ void store16(void *base, size_t vec, u32x4 w) {
  static_cast<u32x4 *>(base)[vec] = w;
}

// ---- wave64 butterflies ----------------------------------------------------
// The first four steps stay inside a 16-lane DPP row (quad swaps, half-row and
// row mirrors); steps 16 and 32 cross rows through the LDS crossbar without
// touching LDS memory.  Every participating lane ends with the full result.
template <int kCtrl> __device__ __forceinline__ float dpp_move(float v) {
  return __int_as_float(
      __builtin_amdgcn_update_dpp(0, __float_as_int(v), kCtrl, 0xF, 0xF, true));
}
template <int kCtrl> __device__ __forceinline__ int dpp_move(int v) {
  return __builtin_amdgcn_update_dpp(0, v, kCtrl, 0xF, 0xF, true);
}
constexpr int kDppSwap1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kDppSwap2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // lane i <-> 7 - i within 8
constexpr int kDppRowMirror = 0x140;   // lane i <-> 15 - i within 16

// Combine across `kLanes` adjacent lanes (4, 8, 16, 32 or 64) with `op`.
template <int kLanes, class V, class Op>
__device__ __forceinline__ V group_reduce(V v, Op op) {
  static_assert(kLanes == 4 || kLanes == 8 || kLanes == 16 || kLanes == 32 || kLanes == 64, "group width");
  v = op(v, v.template moved<kDppSwap1>());
  v = op(v, v.template moved<kDppSwap2>());
  if constexpr (kLanes >= 8) v = op(v, v.template moved<kDppHalfMirror>());
  if constexpr (kLanes >= 16) v = op(v, v.template moved<kDppRowMirror>());
  if constexpr (kLanes >= 32) v = op(v, v.shuffled_xor(16));
  if constexpr (kLanes >= 64) v = op(v, v.shuffled_xor(32));
  return v;
}

struct LaneF32 {
  float x;
  template <int kCtrl> __device__ __forceinline__ LaneF32 moved() const {
    return {dpp_move<kCtrl>(x)};
  }
  __device__ __forceinline__ LaneF32 shuffled_xor(int mask) const {
    return {__shfl_xor(x, mask, kWaveLanes)};
  }
};
struct LaneArg {  // (value, index) candidate of an arg-extremum
  float value;
  int index;
  template <int kCtrl> __device__ __forceinline__ LaneArg moved() const {
    return {dpp_move<kCtrl>(value), dpp_move<kCtrl>(index)};
  }
  __device__ __forceinline__ LaneArg shuffled_xor(int mask) const {
    return {__shfl_xor(value, mask, kWaveLanes), __shfl_xor(index, mask, kWaveLanes)};
  }
};

template <int kLanes> __device__ __forceinline__ float group_sum(float v) {
  return group_reduce<kLanes>(LaneF32{v}, [](LaneF32 a, LaneF32 b) { return LaneF32{a.x + b.x}; }).x;
}
// Plain maximum of NaN-free values.
template <int kLanes> __device__ __forceinline__ float group_max(float v) {
  return group_reduce<kLanes>(LaneF32{v}, [](LaneF32 a, LaneF32 b) {
    return LaneF32{a.x > b.x ? a.x : b.x};
  }).x;
}

// A row handled by `kLanes` adjacent lanes of a block: a slice of a wave, one wave, or
// several whole waves.  Waves of one row meet through `joint` (one float per wave of the
// block) and one block barrier; each call needs its own `joint` array.
template <int kLanes, class Op>
__device__ __forceinline__ float row_reduce(float v, float *joint, Op op) {
  constexpr int kGroup = kLanes < kWaveLanes ? kLanes : kWaveLanes;
  v = group_reduce<kGroup>(LaneF32{v}, [op](LaneF32 a, LaneF32 b) { return LaneF32{op(a.x, b.x)}; }).x;
  if constexpr (kLanes > kWaveLanes) {
    constexpr int kWavesPerRow = kLanes / kWaveLanes;
    if ((threadIdx.x & (kWaveLanes - 1)) == 0) joint[threadIdx.x / kWaveLanes] = v;
    __syncthreads();
    const int first = (threadIdx.x / kLanes) * kWavesPerRow;
    v = joint[first];
#pragma unroll
    for (int w = 1; w < kWavesPerRow; ++w) v = op(v, joint[first + w]);
  }
  return v;
}
template <int kLanes> __device__ __forceinline__ float row_sum(float v, float *joint) {
  return row_reduce<kLanes>(v, joint, [](float a, float b) { return a + b; });
}
template <int kLanes> __device__ __forceinline__ float row_max(float v, float *joint) {
  return row_reduce<kLanes>(v, joint, [](float a, float b) { return a > b ? a : b; });
}
// NaN-propagating extrema of the reference's Reduce
// (src/compute_provider_native/reduction.cc:34-47): the first NaN met sticks;
// +0 ranks above -0 (tests/simd/search_test.cc:203-206).
__device__ __forceinline__ float max_propagate(float a, float b) {
  if (a != a) return a;
  if (b != b) return b;
  if (a == b) return (f32_bits(a) & 0x80000000u) ? b : a;
  return a > b ? a : b;
}
__device__ __forceinline__ float min_propagate(float a, float b) {
  if (a != a) return a;
  if (b != b) return b;
  if (a == b) return (f32_bits(a) & 0x80000000u) ? a : b;
  return a < b ? a : b;
}

// TopK(count = 1, largest) ordering of src/compute_provider_cuda/collectives.cu:478-495:
// a number beats NaN, a larger number beats a smaller one, otherwise (equal,
// -0 vs +0, NaN vs NaN) the lower index wins.  index < 0 marks "no candidate".
__device__ __forceinline__ LaneArg arg_best(LaneArg a, LaneArg b) {
  if (a.index < 0) return b;
  if (b.index < 0) return a;
  const bool a_nan = a.value != a.value, b_nan = b.value != b.value;
  if (a_nan != b_nan) return a_nan ? b : a;
  if (!a_nan && a.value != b.value) return a.value > b.value ? a : b;
  return a.index < b.index ? a : b;
}

}  // namespace hyle_hip
