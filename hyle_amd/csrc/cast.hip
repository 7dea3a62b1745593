// cast.hip -- Cast between storage types and Copy (materialise a strided tensor), for gfx950.
//
// Semantics follow the reference's CPU provider
// (src/compute_provider_native/cast.cc:19-92,225-238 and transform.cc:47-110):
//   float <-> float   decode to f32, encode once (round to nearest even; the codecs of
//                     include/hyle/simd/dtype.h:55-121)
//   int32 -> f32      round to nearest even
//   float -> Bool     truth of the stored magnitude bits: both zeros are false, subnormals,
//                     infinities and NaNs are true
//   Bool  -> float    any nonzero byte is 1, zero is 0
//   equal types       the bytes are kept (Copy)
// The input is any plain tensor (byte strides, elements need not be aligned), the output dense.
#include <type_traits>

#include "device_common.h"
#include "kernels.h"

namespace hyle_hip {
namespace {

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Storage kinds of the cast kernels; Raw* move bytes unchanged.
struct CF32 { static constexpr int kSize = 4; };
struct CF16 { static constexpr int kSize = 2; };
struct CBF16 { static constexpr int kSize = 2; };
struct CBool { static constexpr int kSize = 1; };
struct CI32 { static constexpr int kSize = 4; };
struct CRaw1 { static constexpr int kSize = 1; };
struct CRaw2 { static constexpr int kSize = 2; };
struct CRaw4 { static constexpr int kSize = 4; };

// One element, given its stored bits (zero-extended) -> stored bits of the destination.
template <class S> __device__ __forceinline__ float decode_bits(uint32_t bits) {
  if constexpr (std::is_same_v<S, CF32>) return bits_f32(bits);
  else if constexpr (std::is_same_v<S, CF16>) {
    // The hardware conversion quiets a signalling NaN; the reference's codec keeps the payload
    // as it is (include/hyle/simd/dtype.h:55-70), so infinities and NaNs are widened by hand.
    if ((bits & 0x7C00u) == 0x7C00u)
      return bits_f32(((bits & 0x8000u) << 16) | 0x7F800000u | ((bits & 0x3FFu) << 13));
    return f16_to_f32((uint16_t)bits);
  }
  else if constexpr (std::is_same_v<S, CBF16>) return bits_f32(bits << 16);
  else if constexpr (std::is_same_v<S, CI32>) return (float)(int32_t)bits;  // v_cvt_f32_i32: nearest even
  else return bits != 0 ? 1.0f : 0.0f;  // CBool
}
template <class D> __device__ __forceinline__ uint32_t encode_bits(float v) {
  if constexpr (std::is_same_v<D, CF32>) return f32_bits(v);
  else if constexpr (std::is_same_v<D, CF16>) return f32_to_f16(v);
  else return f32_to_bf16(v);  // CBF16
}
template <class S, class D> __device__ __forceinline__ uint32_t convert_bits(uint32_t bits) {
  if constexpr (std::is_same_v<S, D> || std::is_same_v<D, CRaw1> || std::is_same_v<D, CRaw2> ||
                std::is_same_v<D, CRaw4>) {
    return bits;
  } else if constexpr (std::is_same_v<D, CBool>) {
    constexpr uint32_t kMagnitude = S::kSize == 4 ? 0x7FFFFFFFu : 0x7FFFu;
    return (bits & kMagnitude) != 0 ? 1u : 0u;
  } else {
    return encode_bits<D>(decode_bits<S>(bits));
  }
}

// kCount consecutive elements of kSize bytes packed in 32-bit words.  A lane moves one group per
// step; the group holds 16 / max(source size, destination size) elements, so the wider side is
// one 16-byte access and the narrower side one 8- or 4-byte access, and the lanes of a wave
// touch consecutive memory on both sides with every instruction.
template <int kSize, int kCount> struct Group {
  static constexpr int kWords = kSize * kCount / 4;
  static_assert(kWords == 1 || kWords == 2 || kWords == 4, "a group is 4, 8 or 16 bytes");
  uint32_t w[kWords];
  __device__ __forceinline__ uint32_t get(int i) const {
    if constexpr (kSize == 4) return w[i];
    else if constexpr (kSize == 2) return (w[i / 2] >> (16 * (i % 2))) & 0xFFFFu;
    else return (w[i / 4] >> (8 * (i % 4))) & 0xFFu;
  }
  __device__ __forceinline__ void set(int i, uint32_t bits) {
    if constexpr (kSize == 4) w[i] = bits;
    else if constexpr (kSize == 2) w[i / 2] = i % 2 == 0 ? bits : (w[i / 2] | (bits << 16));
    else w[i / 4] = i % 4 == 0 ? bits : (w[i / 4] | (bits << (8 * (i % 4))));
  }
  __device__ __forceinline__ void load(const void *base, uint32_t group) {
    if constexpr (kWords == 4) {
      const u32x4 a = load16_stream(base, group);
      w[0] = a.x; w[1] = a.y; w[2] = a.z; w[3] = a.w;
    } else if constexpr (kWords == 2) {
      const u32x2 a = __builtin_nontemporal_load(static_cast<const u32x2 *>(base) + group);
      w[0] = a.x; w[1] = a.y;
    } else {
      w[0] = __builtin_nontemporal_load(static_cast<const uint32_t *>(base) + group);
    }
  }
  __device__ __forceinline__ void store(void *base, uint32_t group) const {
    if constexpr (kWords == 4) store16_stream(base, group, u32x4{w[0], w[1], w[2], w[3]});
    else if constexpr (kWords == 2) __builtin_nontemporal_store(u32x2{w[0], w[1]}, static_cast<u32x2 *>(base) + group);
    else __builtin_nontemporal_store(w[0], static_cast<uint32_t *>(base) + group);
  }
  __device__ __forceinline__ void arrived() {
#pragma unroll
    for (int i = 0; i < kWords; ++i) loads_issued(w[i]);
  }
};

template <int kSize> __device__ __forceinline__ uint32_t load_element(const char *p) {
  uint32_t bits = 0;
#pragma unroll
  for (int b = 0; b < kSize; ++b) bits |= (uint32_t)(uint8_t)p[b] << (8 * b);  // any alignment
  return bits;
}
template <int kSize> __device__ __forceinline__ void store_element(void *base, size_t index, uint32_t bits) {
  if constexpr (kSize == 4) static_cast<uint32_t *>(base)[index] = bits;
  else if constexpr (kSize == 2) static_cast<uint16_t *>(base)[index] = (uint16_t)bits;
  else static_cast<uint8_t *>(base)[index] = (uint8_t)bits;
}

template <class S, class D> constexpr int group_elements() {
  return 16 / (S::kSize > D::kSize ? S::kSize : D::kSize);
}

// Dense input, dense output, both 16-byte aligned: a lane converts kUnroll groups, kThreads
// apart.  Loads carry no branches (a lane past the end reads the last group and drops it); the
// groups are taken one after another (kSerial) or all at once, and every store follows the last
// load.
template <class S, class D, int kUnroll, int kThreads, bool kSerial>
__global__ __launch_bounds__(kThreads) void cast_flat(const void *in, void *out, uint32_t groups,
                                                      uint32_t elements) {
  constexpr int kCount = group_elements<S, D>();
  const uint32_t first = blockIdx.x * (kUnroll * kThreads) + threadIdx.x;
  if (groups != 0) {
    Group<S::kSize, kCount> source[kUnroll];
    Group<D::kSize, kCount> result[kUnroll];
    auto load = [&](int k) {
      const uint32_t group = first + k * kThreads;
      source[k].load(in, group < groups ? group : groups - 1);
    };
    auto convert = [&](int k) {
#pragma unroll
      for (int i = 0; i < kCount; ++i) result[k].set(i, convert_bits<S, D>(source[k].get(i)));
    };
    if constexpr (kSerial) {
      load(0);
#pragma unroll
      for (int k = 0; k < kUnroll; ++k) {
        source[k].arrived();
        if (k + 1 < kUnroll) load(k + 1);
        convert(k);
      }
    } else {
#pragma unroll
      for (int k = 0; k < kUnroll; ++k) load(k);
#pragma unroll
      for (int k = 0; k < kUnroll; ++k) source[k].arrived();
#pragma unroll
      for (int k = 0; k < kUnroll; ++k) convert(k);
    }
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      const uint32_t group = first + k * kThreads;
      if (group < groups) result[k].store(out, group);
    }
  }
  // elements past the last whole group
  if (blockIdx.x == 0 && threadIdx.x < kCount) {
    const uint32_t e = groups * kCount + threadIdx.x;
    if (e < elements)
      store_element<D::kSize>(out, e, convert_bits<S, D>(load_element<S::kSize>(static_cast<const char *>(in) + (size_t)e * S::kSize)));
  }
}

// Any strides, any element alignment: one element per lane, the input offset decoded axis by
// axis (src/compute_provider_native/native_plan.h:135-147).
struct CastLayout {
  int32_t rank;
  uint32_t dims[kMaxRank];
  int64_t strides[kMaxRank];
};
template <class S, class D>
__global__ __launch_bounds__(kBlockThreads) void cast_general(const char *in, void *out, uint64_t elements,
                                                              CastLayout layout) {
  const uint64_t e = (uint64_t)blockIdx.x * kBlockThreads + threadIdx.x;
  if (e >= elements) return;
  int64_t offset = 0;
  uint64_t rest = e;
  for (int axis = layout.rank - 1; axis >= 0; --axis) {
    offset += (int64_t)(rest % layout.dims[axis]) * layout.strides[axis];
    rest /= layout.dims[axis];
  }
  store_element<D::kSize>(out, e, convert_bits<S, D>(load_element<S::kSize>(in + offset)));
}

template <int kUnroll, int kThreads, bool kSerial> struct FlatTag {
  static std::string text() {
    return "cast_flat/" + std::to_string(kUnroll) + "x" + std::to_string(kThreads) + (kSerial ? "/serial" : "/batched");
  }
};
struct GeneralTag {
  static std::string text() { return "cast_general"; }
};

template <class S, class D, int kUnroll, int kThreads, bool kSerial>
hipError_t run_flat_as(const void *in, void *out, uint64_t elements, hipStream_t s) {
  const uint64_t groups = elements / group_elements<S, D>();
  const uint64_t per_block = (uint64_t)kUnroll * kThreads;
  uint64_t blocks = (groups + per_block - 1) / per_block;
  if (blocks == 0) blocks = 1;  // the tail still needs block 0
  note_variant<FlatTag<kUnroll, kThreads, kSerial>>();
  hipLaunchKernelGGL((cast_flat<S, D, kUnroll, kThreads, kSerial>), dim3((uint32_t)blocks), dim3(kThreads), 0, s,
                     in, out, (uint32_t)groups, (uint32_t)elements);
  return hipGetLastError();
}

template <class S, class D>
hipError_t run_pair(const CastParams &p, const void *in, void *out, bool vectorised, hipStream_t s) {
  if (p.dense_input && vectorised) {
    // Launch shape from the traffic, as for the elementwise kernels: fat blocks that take their
    // groups one after another below about 110 MB, several groups at once per lane above.
    const uint64_t traffic = p.elements * (uint64_t)(S::kSize + D::kSize);
    // Measured on MI355X, [8192, 2048]: f32 -> bf16 16.6 us and bf16 -> f32 17.3 us with 8
    // groups per lane taken serially in blocks of 512 threads, against 18.9 / 17.6 us with one
    // group per lane; a 201 MB copy 32.6 us with one group per lane against 35-37 us serially.
    if (traffic > (110ull << 20)) return run_flat_as<S, D, 1, 256, false>(in, out, p.elements, s);
    if (traffic > (48ull << 20)) return run_flat_as<S, D, 8, 512, true>(in, out, p.elements, s);
    return run_flat_as<S, D, 4, 512, true>(in, out, p.elements, s);
  }
  CastLayout layout{};
  layout.rank = p.rank;
  for (int i = 0; i < kMaxRank; ++i) {
    layout.dims[i] = p.dims[i];
    layout.strides[i] = p.strides[i];
  }
  const uint64_t blocks = (p.elements + kBlockThreads - 1) / kBlockThreads;
  note_variant<GeneralTag>();
  hipLaunchKernelGGL((cast_general<S, D>), dim3((uint32_t)blocks), dim3(kBlockThreads), 0, s,
                     static_cast<const char *>(in), out, p.elements, layout);
  return hipGetLastError();
}

template <class S>
hipError_t run_from(const CastParams &p, const void *in, void *out, bool vectorised, hipStream_t s) {
  switch (p.dst) {
    case CastType::kF32:
      if constexpr (!std::is_same_v<S, CF32>) return run_pair<S, CF32>(p, in, out, vectorised, s);
      break;
    case CastType::kF16:
      if constexpr (!std::is_same_v<S, CF16> && !std::is_same_v<S, CI32>) return run_pair<S, CF16>(p, in, out, vectorised, s);
      break;
    case CastType::kBF16:
      if constexpr (!std::is_same_v<S, CBF16> && !std::is_same_v<S, CI32>) return run_pair<S, CBF16>(p, in, out, vectorised, s);
      break;
    case CastType::kBool:
      if constexpr (!std::is_same_v<S, CBool> && !std::is_same_v<S, CI32>) return run_pair<S, CBool>(p, in, out, vectorised, s);
      break;
    default: break;
  }
  return hipErrorInvalidValue;
}

}  // namespace

hipError_t launch_cast(const CastParams &p, const void *in, void *out, bool vectorised, hipStream_t stream) {
  if (p.elements == 0) return hipSuccess;
  if (p.copy_size != 0) {
    // A dense copy is a stream of bytes whatever the element type: whole 4-byte words when the
    // byte count allows, so that a lane moves 16 bytes per step.
    const uint64_t bytes = p.elements * p.copy_size;
    if (p.dense_input && vectorised && bytes % 4 == 0) {
      CastParams words = p;
      words.elements = bytes / 4;
      return run_pair<CRaw4, CRaw4>(words, in, out, true, stream);
    }
    switch (p.copy_size) {
      case 1: return run_pair<CRaw1, CRaw1>(p, in, out, vectorised, stream);
      case 2: return run_pair<CRaw2, CRaw2>(p, in, out, vectorised, stream);
      case 4: return run_pair<CRaw4, CRaw4>(p, in, out, vectorised, stream);
      default: return hipErrorInvalidValue;
    }
  }
  switch (p.src) {
    case CastType::kF32: return run_from<CF32>(p, in, out, vectorised, stream);
    case CastType::kF16: return run_from<CF16>(p, in, out, vectorised, stream);
    case CastType::kBF16: return run_from<CBF16>(p, in, out, vectorised, stream);
    case CastType::kBool: return run_from<CBool>(p, in, out, vectorised, stream);
    case CastType::kI32: return run_from<CI32>(p, in, out, vectorised, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace hyle_hip
