/*
 * hyle_oracle.c -- CPU restatement of the reference's scalar semantics for the
 * tensor hot path.  TEST INFRASTRUCTURE ONLY (see hyle_oracle.h): the shipped
 * library never links, loads or calls this file.
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math (see oracle/Makefile).
 */
#include "hyle_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------ */
/* bit helpers                                                              */
/* ------------------------------------------------------------------------ */
static inline float bits_to_f32(uint32_t b) {
  float f;
  memcpy(&f, &b, sizeof f);
  return f;
}
static inline uint32_t f32_to_bits(float f) {
  uint32_t b;
  memcpy(&b, &f, sizeof b);
  return b;
}

/* ------------------------------------------------------------------------ */
/* codecs: include/hyle/simd/dtype.h:55-121                                 */
/* ------------------------------------------------------------------------ */

/* include/hyle/simd/dtype.h:55-67.  Subnormals: mantissa * 2^-24 (exact). */
float hyle_oracle_f16_to_f32(uint16_t h) {
  const uint32_t sign = (uint32_t)h >> 15;
  const uint32_t exp5 = ((uint32_t)h >> 10) & 0x1Fu;
  const uint32_t man = (uint32_t)h & 0x3FFu;
  if (exp5 == 0) {
    const float sub = (1.0f / 16384) * ((float)man * (1.0f / 1024));
    return sign ? -sub : sub;
  }
  const uint32_t exp8 = (exp5 == 31) ? 0xFFu : exp5 + (127 - 15);
  return bits_to_f32((sign << 31) | (exp8 << 23) | (man << 13));
}

/* include/hyle/simd/dtype.h:72-101.  RN-even through an odd-bit + (half-ulp-1)
 * bias; overflow -> inf; NaN -> mantissa 0x3FF. */
uint16_t hyle_oracle_f32_to_f16(float f) {
  const uint32_t u = f32_to_bits(f);
  const uint32_t sign = u >> 31;
  const uint32_t exp8 = (u >> 23) & 0xFFu;
  const uint32_t man = u & 0x7FFFFFu;

  int idx = 126 - (int)exp8;
  if (idx < 13) idx = 13;
  if (idx > 24) idx = 24;
  const uint32_t odd = ((man | 0x800000u) >> idx) & 1u;
  const uint32_t rounded = man + odd + (1u << (idx - 1)) - 1u;
  const int carry = rounded >= (1u << 23);
  const int exp = (int)exp8 - 127 + (carry ? 1 : 0);

  if (exp < -24) return (uint16_t)(sign << 15);

  const int is_nan = (exp8 == 255) && (man != 0);
  const int overflowed = exp >= 16;
  int be16 = exp + 15;
  if (be16 < 0) be16 = 0;
  if (be16 > 31) be16 = 31;
  const int sub_exp = (-14 - exp) > 0 ? (-14 - exp) : 0;
  const uint32_t shifted = (rounded & 0x7FFFFFu) >> (13 + sub_exp);
  const uint32_t leading = (sub_exp == 0) ? 0u : (1024u >> sub_exp);
  const uint32_t man16 = is_nan ? 0x3FFu : (overflowed ? 0u : leading + shifted);
  return (uint16_t)((sign << 15) | ((uint32_t)be16 << 10) | man16);
}

/* include/hyle/simd/dtype.h:107-109 */
float hyle_oracle_bf16_to_f32(uint16_t b) {
  return bits_to_f32((uint32_t)b << 16);
}

/* include/hyle/simd/dtype.h:114-121.  RN-even for finite input, truncation for
 * inf/NaN, NaN keeps its upper payload and gets bit 6 set. */
uint16_t hyle_oracle_f32_to_bf16(float f) {
  const uint32_t u = f32_to_bits(f);
  const uint32_t mag = u & 0x7FFFFFFFu;
  const uint32_t incr = (mag < 0x7F800000u) ? (0x7FFFu + ((u >> 16) & 1u)) : 0u;
  const uint32_t quiet = (mag > 0x7F800000u) ? (1u << 6) : 0u;
  return (uint16_t)(quiet | ((u + incr) >> 16));
}

static inline size_t type_size(int type) {
  return type == HYLE_ORACLE_F32 || type == HYLE_ORACLE_I32 ? 4u : 2u;
}

/* src/compute_provider_native/numeric.h:13-47 (decode / encode / load / store) */
static inline float load_as_f32(int type, const void *p) {
  if (type == HYLE_ORACLE_F32) {
    float v;
    memcpy(&v, p, 4);
    return v;
  }
  uint16_t h;
  memcpy(&h, p, 2);
  return type == HYLE_ORACLE_F16 ? hyle_oracle_f16_to_f32(h)
                                 : hyle_oracle_bf16_to_f32(h);
}
static inline void store_from_f32(int type, void *p, float v) {
  if (type == HYLE_ORACLE_F32) {
    memcpy(p, &v, 4);
    return;
  }
  const uint16_t h = type == HYLE_ORACLE_F16 ? hyle_oracle_f32_to_f16(v)
                                             : hyle_oracle_f32_to_bf16(v);
  memcpy(p, &h, 2);
}

void hyle_oracle_convert_to_f32(int type, const void *src, float *dst,
                                size_t n) {
  const unsigned char *s = (const unsigned char *)src;
  const size_t w = type_size(type);
  for (size_t i = 0; i < n; ++i) dst[i] = load_as_f32(type, s + i * w);
}
void hyle_oracle_convert_from_f32(int type, const float *src, void *dst,
                                  size_t n) {
  unsigned char *d = (unsigned char *)dst;
  const size_t w = type_size(type);
  for (size_t i = 0; i < n; ++i) store_from_f32(type, d + i * w, src[i]);
}

/* ------------------------------------------------------------------------ */
/* shapes                                                                   */
/* ------------------------------------------------------------------------ */

/* src/compute_ops/operation.cc:249-278: NumPy right-aligned broadcasting. */
int hyle_oracle_broadcast_shape(const int64_t *left, int left_rank,
                                const int64_t *right, int right_rank,
                                int64_t *out) {
  const int rank = left_rank > right_rank ? left_rank : right_rank;
  if (rank > HYLE_ORACLE_MAX_RANK) return -1;
  for (int reverse = 0; reverse < rank; ++reverse) {
    const int64_t l = reverse < left_rank ? left[left_rank - 1 - reverse] : 1;
    const int64_t r = reverse < right_rank ? right[right_rank - 1 - reverse] : 1;
    int64_t extent;
    if (l == r)
      extent = l;
    else if (l == 1)
      extent = r;
    else if (r == 1)
      extent = l;
    else
      return -1;
    out[rank - 1 - reverse] = extent;
  }
  return rank;
}

/* src/compute_provider_native/native_plan.h:152-174: walk the dense output
 * coordinate from the innermost axis; an input axis of extent 1 (or a missing
 * leading axis) contributes nothing. */
size_t hyle_oracle_broadcast_byte_offset(const int64_t *in_dims,
                                         const int64_t *in_strides, int in_rank,
                                         const int64_t *out_dims, int out_rank,
                                         size_t linear) {
  size_t offset = 0;
  for (int reverse = 0; reverse < out_rank; ++reverse) {
    const int out_axis = out_rank - 1 - reverse;
    const size_t extent = (size_t)out_dims[out_axis];
    const size_t coordinate = linear % extent;
    linear /= extent;
    if (reverse >= in_rank) continue;
    const int in_axis = in_rank - 1 - reverse;
    if (in_dims[in_axis] != 1) offset += coordinate * (size_t)in_strides[in_axis];
  }
  return offset;
}

/* src/compute_provider_native/native_plan.h:135-147 */
size_t hyle_oracle_logical_byte_offset(const int64_t *dims,
                                       const int64_t *strides, int rank,
                                       size_t linear) {
  size_t offset = 0;
  for (int reverse = 0; reverse < rank; ++reverse) {
    const int axis = rank - 1 - reverse;
    const size_t extent = (size_t)dims[axis];
    offset += (linear % extent) * (size_t)strides[axis];
    linear /= extent;
  }
  return offset;
}

static size_t element_count(const int64_t *dims, int rank) {
  size_t n = 1;
  for (int i = 0; i < rank; ++i) n *= (size_t)dims[i];
  return n;
}

/* ------------------------------------------------------------------------ */
/* elementwise                                                              */
/* ------------------------------------------------------------------------ */

/* src/compute_provider_native/elementwise.cc:102-114 gives Add / Subtract /
 * Divide / Minimum; Multiply and Maximum follow the reference's own test
 * oracle (tests/compute_provider_native/elementwise_test.cc:84-101) and the
 * CUDA tensor kernel (src/compute_provider_cuda/tensor_kernel.cu:150-165). */
float hyle_oracle_binary_scalar(int kind, float l, float r) {
  switch (kind) {
    case HYLE_ORACLE_ADD: return l + r;
    case HYLE_ORACLE_SUBTRACT: return l - r;
    case HYLE_ORACLE_MULTIPLY: return l * r;
    case HYLE_ORACLE_DIVIDE: return l / r;
    case HYLE_ORACLE_MINIMUM: return fminf(l, r);
    case HYLE_ORACLE_MAXIMUM: return fmaxf(l, r);
    default: return NAN;
  }
}

/* src/compute_provider_native/elementwise.cc:349-366 (per-element route; the
 * linear and chunked routes compute the same values). */
void hyle_oracle_binary(int kind, int type, const void *left,
                        const int64_t *ld, const int64_t *ls, int lr,
                        const void *right, const int64_t *rd, const int64_t *rs,
                        int rr, void *out, const int64_t *od, int orank) {
  const size_t n = element_count(od, orank);
  const size_t w = type_size(type);
  const unsigned char *a = (const unsigned char *)left;
  const unsigned char *b = (const unsigned char *)right;
  unsigned char *o = (unsigned char *)out;
  for (size_t i = 0; i < n; ++i) {
    const float x = load_as_f32(
        type, a + hyle_oracle_broadcast_byte_offset(ld, ls, lr, od, orank, i));
    const float y = load_as_f32(
        type, b + hyle_oracle_broadcast_byte_offset(rd, rs, rr, od, orank, i));
    store_from_f32(type, o + i * w, hyle_oracle_binary_scalar(kind, x, y));
  }
}

void hyle_oracle_binary_chain(int kind0, int kind1, int type, const void *a,
                              const int64_t *ad, const int64_t *as, int ar,
                              const void *b, const int64_t *bd,
                              const int64_t *bs, int br, const void *c,
                              const int64_t *cd, const int64_t *cs, int cr,
                              void *out, const int64_t *od, int orank) {
  const size_t n = element_count(od, orank);
  const size_t w = type_size(type);
  const unsigned char *pa = (const unsigned char *)a;
  const unsigned char *pb = (const unsigned char *)b;
  const unsigned char *pc = (const unsigned char *)c;
  unsigned char *o = (unsigned char *)out;
  for (size_t i = 0; i < n; ++i) {
    const float x = load_as_f32(
        type, pa + hyle_oracle_broadcast_byte_offset(ad, as, ar, od, orank, i));
    const float y = load_as_f32(
        type, pb + hyle_oracle_broadcast_byte_offset(bd, bs, br, od, orank, i));
    const float z = load_as_f32(
        type, pc + hyle_oracle_broadcast_byte_offset(cd, cs, cr, od, orank, i));
    /* the intermediate passes through the storage type, exactly as two
     * separately submitted Binary operations would leave it */
    unsigned char tmp[4];
    store_from_f32(type, tmp, hyle_oracle_binary_scalar(kind0, x, y));
    const float t = load_as_f32(type, tmp);
    store_from_f32(type, o + i * w, hyle_oracle_binary_scalar(kind1, t, z));
  }
}

/* src/simd/math/activations.cc:21-25 */
float hyle_oracle_sigmoid(float x) {
  if (isnan(x)) return x;
  const float e = expf(-fabsf(x));
  return x < 0.0f ? e / (1.0f + e) : 1.0f / (1.0f + e);
}

/* src/simd/math/activations.cc:44-47 */
float hyle_oracle_silu(float x) {
  if (x == -INFINITY) return 0.0f;
  return x * hyle_oracle_sigmoid(x);
}

/* src/simd/math/activations.cc:106-112 */
void hyle_oracle_silu_rows(int type, const void *src, void *dst, size_t n) {
  const unsigned char *s = (const unsigned char *)src;
  unsigned char *d = (unsigned char *)dst;
  const size_t w = type_size(type);
  for (size_t i = 0; i < n; ++i)
    store_from_f32(type, d + i * w, hyle_oracle_silu(load_as_f32(type, s + i * w)));
}

/* src/simd/math/activations.cc:114-122 */
void hyle_oracle_swiglu(int type, const void *gate, const void *value,
                        void *dst, size_t n) {
  const unsigned char *g = (const unsigned char *)gate;
  const unsigned char *v = (const unsigned char *)value;
  unsigned char *d = (unsigned char *)dst;
  const size_t w = type_size(type);
  for (size_t i = 0; i < n; ++i) {
    const float gv = load_as_f32(type, g + i * w);
    const float lv = load_as_f32(type, v + i * w);
    store_from_f32(type, d + i * w, hyle_oracle_silu(gv) * lv);
  }
}

/* ---- every Unary kind and the three gate activations -------------------- */
/* src/simd/math/activations.cc:27-41 */
static float gelu_erf(float x) {
  if (x == -INFINITY) return 0.0f;
  return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f));
}
static float gelu_tanh(float x) {
  if (x == -INFINITY) return 0.0f;
  const float inner = 0.79788456080286535588f * x * fmaf(0.044715f, x * x, 1.0f);
  return 0.5f * x * (1.0f + tanhf(inner));
}

/* UnaryKind order of include/hyle/compute/operation.h:57-73.  neg, exp, log,
 * sqrt, rsqrt, tanh, relu, silu: src/compute_provider_native/elementwise.cc:30-55;
 * sigmoid, gelu, gelu_tanh: src/simd/math/activations.cc:21-41; abs and
 * softplus (evaluated in double): tests/compute_provider_native/elementwise_test.cc:43-82.
 * exp, log, tanh, erf are the host libm's. */
float hyle_oracle_unary_scalar(int kind, float x) {
  switch (kind) {
    case 0: return fabsf(x);
    case 1: return -x;
    case 2: return expf(x);
    case 3: return logf(x);
    case 4: return sqrtf(x);
    case 5: return 1.0f / sqrtf(x);
    case 6: return tanhf(x);
    case 7: return hyle_oracle_sigmoid(x);
    case 8: return isnan(x) ? x : (x > 0.0f ? x : 0.0f);
    case 9: return gelu_erf(x);
    case 10: return gelu_tanh(x);
    case 11: return hyle_oracle_silu(x);
    default: return (float)log1p(exp((double)x));
  }
}

/* decode -> f32 function -> one rounding
 * (src/compute_provider_native/elementwise.cc:83-99, src/simd/math/activations.cc:106-112) */
void hyle_oracle_unary(int kind, int type, const void *src, void *dst, size_t n) {
  const unsigned char *s = (const unsigned char *)src;
  unsigned char *d = (unsigned char *)dst;
  const size_t w = type_size(type);
  for (size_t i = 0; i < n; ++i)
    store_from_f32(type, d + i * w, hyle_oracle_unary_scalar(kind, load_as_f32(type, s + i * w)));
}

/* src/simd/math/activations.cc:114-122 with activation = silu (0), gelu (1),
 * gelu_tanh (2): GatedActivationKind of include/hyle/compute/operation.h:91-95 */
void hyle_oracle_gated(int activation, int type, const void *gate, const void *value,
                       void *dst, size_t n) {
  const unsigned char *g = (const unsigned char *)gate;
  const unsigned char *v = (const unsigned char *)value;
  unsigned char *d = (unsigned char *)dst;
  const size_t w = type_size(type);
  for (size_t i = 0; i < n; ++i) {
    const float gv = load_as_f32(type, g + i * w);
    const float lv = load_as_f32(type, v + i * w);
    const float a = activation == 0 ? hyle_oracle_silu(gv) : (activation == 1 ? gelu_erf(gv) : gelu_tanh(gv));
    store_from_f32(type, d + i * w, a * lv);
  }
}

/* src/compute_provider_native/elementwise.cc:192-208: value = gate + hidden */
void hyle_oracle_swiglu_packed(int type, const void *packed, void *dst,
                               size_t rows, size_t hidden) {
  const unsigned char *p = (const unsigned char *)packed;
  unsigned char *d = (unsigned char *)dst;
  const size_t w = type_size(type);
  for (size_t r = 0; r < rows; ++r) {
    const unsigned char *gate = p + r * 2 * hidden * w;
    hyle_oracle_swiglu(type, gate, gate + hidden * w, d + r * hidden * w, hidden);
  }
}

/* ------------------------------------------------------------------------ */
/* RMSNorm                                                                  */
/* ------------------------------------------------------------------------ */

/* src/simd/math/activations.cc:124-146 */
void hyle_oracle_rms_norm_row(int type, int weight_type, const void *src,
                              const void *weight, void *dst, size_t n,
                              float epsilon) {
  if (n == 0) return;
  const unsigned char *s = (const unsigned char *)src;
  const unsigned char *wp = (const unsigned char *)weight;
  unsigned char *d = (unsigned char *)dst;
  const size_t w = type_size(type);
  const size_t ww = type_size(weight_type);
  float sum_squares = 0.0f;
  for (size_t i = 0; i < n; ++i) {
    const float v = load_as_f32(type, s + i * w);
    sum_squares = fmaf(v, v, sum_squares);
  }
  const float inverse_rms = 1.0f / sqrtf(sum_squares / (float)n + epsilon);
  if (weight == NULL) {
    for (size_t i = 0; i < n; ++i)
      store_from_f32(type, d + i * w, load_as_f32(type, s + i * w) * inverse_rms);
  } else {
    for (size_t i = 0; i < n; ++i) {
      const float v = load_as_f32(type, s + i * w);
      const float scale = load_as_f32(weight_type, wp + i * ww);
      store_from_f32(type, d + i * w, v * inverse_rms * scale);
    }
  }
}

void hyle_oracle_rms_norm(int type, int weight_type, const void *src,
                          const void *weight, void *dst, size_t rows,
                          size_t hidden, float epsilon) {
  const unsigned char *s = (const unsigned char *)src;
  unsigned char *d = (unsigned char *)dst;
  const size_t w = type_size(type);
  for (size_t r = 0; r < rows; ++r)
    hyle_oracle_rms_norm_row(type, weight_type, s + r * hidden * w, weight,
                             d + r * hidden * w, hidden, epsilon);
}

/* src/simd/math/activations.cc:148-175: mean from a plain running sum, centred
 * squares through an fma chain, inverse = 1 / sqrt(ss / n + eps); without
 * parameters (x - mean) * inverse, with them fma(normalised, scale, bias).
 * The scalar floor has no scale-only form; the provider level defines it as
 * normalised * scale (tests/compute_provider_native/normalization_test.cc:69-127). */
void hyle_oracle_layer_norm_row(int type, int param_type, const void *src,
                                const void *scale, const void *bias, void *dst,
                                size_t n, float epsilon) {
  if (n == 0) return;
  const unsigned char *s = (const unsigned char *)src;
  const unsigned char *sp = (const unsigned char *)scale;
  const unsigned char *bp = (const unsigned char *)bias;
  unsigned char *d = (unsigned char *)dst;
  const size_t w = type_size(type);
  const size_t pw = type_size(param_type);
  float sum = 0.0f;
  for (size_t i = 0; i < n; ++i) sum += load_as_f32(type, s + i * w);
  const float mean = sum / (float)n;
  float sum_squares = 0.0f;
  for (size_t i = 0; i < n; ++i) {
    const float centered = load_as_f32(type, s + i * w) - mean;
    sum_squares = fmaf(centered, centered, sum_squares);
  }
  const float inverse = 1.0f / sqrtf(sum_squares / (float)n + epsilon);
  for (size_t i = 0; i < n; ++i) {
    const float normalized = (load_as_f32(type, s + i * w) - mean) * inverse;
    if (scale == NULL)
      store_from_f32(type, d + i * w, normalized);
    else if (bias == NULL)
      store_from_f32(type, d + i * w,
                     normalized * load_as_f32(param_type, sp + i * pw));
    else
      store_from_f32(type, d + i * w,
                     fmaf(normalized, load_as_f32(param_type, sp + i * pw),
                          load_as_f32(param_type, bp + i * pw)));
  }
}

void hyle_oracle_layer_norm(int type, int param_type, const void *src,
                            const void *scale, const void *bias, void *dst,
                            size_t rows, size_t hidden, float epsilon) {
  const unsigned char *s = (const unsigned char *)src;
  unsigned char *d = (unsigned char *)dst;
  const size_t w = type_size(type);
  for (size_t r = 0; r < rows; ++r)
    hyle_oracle_layer_norm_row(type, param_type, s + r * hidden * w, scale, bias,
                               d + r * hidden * w, hidden, epsilon);
}

/* src/compute_provider_native/normalization.cc:41-80.  The reference sums each
 * tile with simd::dot (a Highway vector dot: lane order is target-dependent),
 * here each tile is summed in index order without fusing; the row total adds
 * tile sums in tile order as the reference does.  Parity of the tile-internal
 * order is unpinned at the bit level. */
void hyle_oracle_rms_norm_native(int type, int weight_type, const void *src,
                                 const void *weight, void *dst, size_t rows,
                                 size_t hidden, float epsilon) {
  const unsigned char *s = (const unsigned char *)src;
  const unsigned char *wp = (const unsigned char *)weight;
  unsigned char *d = (unsigned char *)dst;
  const size_t w = type_size(type);
  const size_t ww = type_size(weight_type);
  float values[128];
  if (hidden == 0) return;
  for (size_t r = 0; r < rows; ++r) {
    const unsigned char *row = s + r * hidden * w;
    unsigned char *out = d + r * hidden * w;
    float squares = 0.0f;
    for (size_t c = 0; c < hidden; c += 128) {
      const size_t size = hidden - c < 128 ? hidden - c : 128;
      float tile = 0.0f;
      for (size_t i = 0; i < size; ++i) {
        const float v = load_as_f32(type, row + (c + i) * w);
        tile += v * v;
      }
      squares += tile;
    }
    const float inverse = 1.0f / sqrtf(squares / (float)hidden + epsilon);
    for (size_t c = 0; c < hidden; c += 128) {
      const size_t size = hidden - c < 128 ? hidden - c : 128;
      for (size_t i = 0; i < size; ++i)
        values[i] = (load_as_f32(type, row + (c + i) * w) - 0.0f) * inverse;
      if (weight != NULL) {
        for (size_t i = 0; i < size; ++i)
          values[i] = values[i] * load_as_f32(weight_type, wp + (c + i) * ww);
      }
      for (size_t i = 0; i < size; ++i)
        store_from_f32(type, out + (c + i) * w, values[i]);
    }
  }
}

/* ------------------------------------------------------------------------ */
/* softmax                                                                  */
/* ------------------------------------------------------------------------ */

/* src/simd/math/activations.cc:177-192 */
static int finite_row_max(const float *src, size_t n, float *maximum) {
  float m = -INFINITY;
  for (size_t i = 0; i < n; ++i) {
    const float x = src[i];
    if (isnan(x) || x == INFINITY) {
      *maximum = m;
      return 0;
    }
    if (x > m) m = x;
  }
  *maximum = m;
  return isfinite(m);
}

/* src/simd/math/activations.cc:301-317: invalid row (any NaN, any +inf, or no
 * finite maximum) becomes all quiet NaN; the exp sum is accumulated in double
 * and the row scaled by float(1/sum). */
void hyle_oracle_softmax_f32_row(const float *src, float *dst, size_t n) {
  if (n == 0) return;
  float maximum = 0.0f;
  if (!finite_row_max(src, n, &maximum)) {
    for (size_t i = 0; i < n; ++i) dst[i] = NAN;
    return;
  }
  double sum = 0.0;
  for (size_t i = 0; i < n; ++i) {
    const float value = expf(src[i] - maximum);
    dst[i] = value;
    sum += (double)value;
  }
  const float inverse = (float)(1.0 / sum);
  for (size_t i = 0; i < n; ++i) dst[i] *= inverse;
}

/* src/compute_provider_native/transformer.cc:44-57 (bool mask) and 165-191 (row
 * loop over a dense last axis); additive mask per
 * src/compute_provider_cuda/reduction_kernel.cu:130-146. */
/* LogSoftmax of one row, src/compute_provider_cuda/reduction_kernel.cu:73-86,
 * 148-196: the maximum is the first NaN, else the largest value at its lowest
 * column; that one column is left out of the f32 sum of exp(v - max) so that
 * log1p keeps small tails (the sum in the kernel's own order: strided partial
 * sums of 256 threads, then a tree); a maximum that is not finite makes the row NaN;
 * result (v - max) - log1p(sum). */
void hyle_oracle_log_softmax_f32_row(const float *src, float *dst, size_t n) {
  if (n == 0) return;
  size_t chosen = 0;
  for (size_t i = 1; i < n; ++i) {
    if (isnan(src[chosen])) break;
    if (isnan(src[i]) || src[i] > src[chosen]) chosen = i;
  }
  const float maximum = src[chosen];
  /* the kernel's order: 256 threads add every 256th column, a tree joins them */
  float partial[256];
  for (size_t t = 0; t < 256; ++t) {
    partial[t] = 0.0f;
    for (size_t i = t; i < n; i += 256)
      if (i != chosen) partial[t] += expf(src[i] - maximum);
  }
  for (size_t half = 128; half > 0; half >>= 1)
    for (size_t t = 0; t < half; ++t) partial[t] += partial[t + half];
  const float sum = partial[0];
  const float normalizer = isfinite(maximum) ? log1pf(sum) : NAN;
  for (size_t i = 0; i < n; ++i) dst[i] = (src[i] - maximum) - normalizer;
}

/* LogSoftmax of one row as the reference's scalar floor writes it
 * (src/simd/math/activations.cc:320-336): the same row validity rule as softmax
 * (any NaN, any +inf or nothing above -inf: the whole row is a quiet NaN), the
 * sum of expf(v - max) in double, shift = max + (float)log(sum), result
 * v - shift. */
void hyle_oracle_log_softmax_floor_f32_row(const float *src, float *dst, size_t n) {
  if (n == 0) return;
  float maximum = -INFINITY;
  int valid = 1;
  for (size_t i = 0; i < n && valid; ++i) {
    if (isnan(src[i]) || src[i] == INFINITY) valid = 0;
    else if (src[i] > maximum) maximum = src[i];
  }
  if (!valid || !isfinite(maximum)) {
    for (size_t i = 0; i < n; ++i) dst[i] = NAN;
    return;
  }
  double sum = 0.0;
  for (size_t i = 0; i < n; ++i) sum += (double)expf(src[i] - maximum);
  const float shift = maximum + (float)log(sum);
  for (size_t i = 0; i < n; ++i) dst[i] = src[i] - shift;
}

static void softmax_rows(int log_form, int type, const void *src, void *dst,
                         const int64_t *in_dims, int in_rank, float scale,
                         int mask_kind, const void *mask,
                         const int64_t *mask_dims, const int64_t *mask_strides,
                         int mask_rank) {
  if (in_rank <= 0) return;
  const size_t width = (size_t)in_dims[in_rank - 1];
  const size_t total = element_count(in_dims, in_rank);
  if (total == 0 || width == 0) return;
  const size_t rows = total / width;
  const size_t w = type_size(type);
  const unsigned char *s = (const unsigned char *)src;
  const unsigned char *m = (const unsigned char *)mask;
  unsigned char *d = (unsigned char *)dst;
  float *scratch = (float *)malloc(width * sizeof(float));
  if (scratch == NULL) return;
  for (size_t r = 0; r < rows; ++r) {
    for (size_t lane = 0; lane < width; ++lane) {
      const size_t logical = r * width + lane;
      float value = load_as_f32(type, s + logical * w);
      value *= scale;
      if (mask_kind == HYLE_ORACLE_MASK_BOOLEAN) {
        const size_t off = hyle_oracle_broadcast_byte_offset(
            mask_dims, mask_strides, mask_rank, in_dims, in_rank, logical);
        if (m[off] == 0) value = -INFINITY;
      } else if (mask_kind == HYLE_ORACLE_MASK_ADDITIVE) {
        const size_t off = hyle_oracle_broadcast_byte_offset(
            mask_dims, mask_strides, mask_rank, in_dims, in_rank, logical);
        value = value + load_as_f32(type, m + off);
      }
      scratch[lane] = value;
    }
    if (log_form) hyle_oracle_log_softmax_f32_row(scratch, scratch, width);
    else hyle_oracle_softmax_f32_row(scratch, scratch, width);
    for (size_t lane = 0; lane < width; ++lane)
      store_from_f32(type, d + (r * width + lane) * w, scratch[lane]);
  }
  free(scratch);
}

void hyle_oracle_softmax(int type, const void *src, void *dst,
                         const int64_t *in_dims, int in_rank, float scale,
                         int mask_kind, const void *mask,
                         const int64_t *mask_dims, const int64_t *mask_strides,
                         int mask_rank) {
  softmax_rows(0, type, src, dst, in_dims, in_rank, scale, mask_kind, mask, mask_dims,
               mask_strides, mask_rank);
}

void hyle_oracle_log_softmax(int type, const void *src, void *dst,
                             const int64_t *in_dims, int in_rank, float scale,
                             int mask_kind, const void *mask,
                             const int64_t *mask_dims, const int64_t *mask_strides,
                             int mask_rank) {
  softmax_rows(1, type, src, dst, in_dims, in_rank, scale, mask_kind, mask, mask_dims,
               mask_strides, mask_rank);
}

/* ------------------------------------------------------------------------ */
/* reductions                                                               */
/* ------------------------------------------------------------------------ */

/* src/compute_provider_native/reduction.cc:24-47: once the running extremum is
 * NaN it stays NaN; a NaN input replaces a non-NaN running value.  Equal values
 * of opposite sign follow the row primitive the dense route calls
 * (simd::max_value / simd::min_value, pinned by tests/simd/search_test.cc:196-206):
 * the maximum of {-0, +0} is +0 and the minimum is -0, whatever the order. */
static void accumulate_extremum(int maximum, float value, float *result) {
  if (isnan(*result)) return;
  if (isnan(value)) {
    *result = value;
    return;
  }
  if (value == *result) {
    if (maximum ? !signbit(value) : signbit(value)) *result = value;
    return;
  }
  if (maximum ? value > *result : value < *result) *result = value;
}

void hyle_oracle_reduce_last_axis(int kind, int type, const void *src,
                                  void *dst, size_t rows, size_t width) {
  const unsigned char *s = (const unsigned char *)src;
  unsigned char *d = (unsigned char *)dst;
  const size_t w = type_size(type);
  for (size_t r = 0; r < rows; ++r) {
    const unsigned char *row = s + r * width * w;
    float result;
    if (kind == HYLE_ORACLE_MIN || kind == HYLE_ORACLE_MAX) {
      const int maximum = kind == HYLE_ORACLE_MAX;
      result = maximum ? -INFINITY : INFINITY;
      for (size_t i = 0; i < width; ++i)
        accumulate_extremum(maximum, load_as_f32(type, row + i * w), &result);
    } else {
      /* src/compute_provider_cuda/reduction_kernel.cu:92-116: f32 accumulate;
       * the summation order is unspecified there (tolerance-compared). */
      float sum = 0.0f;
      for (size_t i = 0; i < width; ++i) sum += load_as_f32(type, row + i * w);
      result = sum;
      if (kind == HYLE_ORACLE_MEAN)
        result = width == 0 ? NAN : sum / (float)width;
    }
    store_from_f32(type, d + r * w, result);
  }
}

/* Reduce over any set of axes of a strided tensor.  Coordinates as in
 * src/compute_provider_cuda/reduction_kernel.cu:38-48 (the result index runs
 * row-major over the axes that are kept, the folded index row-major over the
 * reduced ones; byte strides, any alignment), one result per output element
 * as in :88-113 (f32 accumulation in the order of the folded index; mean =
 * sum / count, NaN for an empty reduction; identities 0, +inf, -inf).  The
 * same walk is src/compute_provider_native/reduction.cc:82-111. */
void hyle_oracle_reduce(int kind, int type, const void *src, int rank,
                        const int64_t *dims, const int64_t *byte_strides,
                        uint32_t axes_mask, void *dst) {
  const unsigned char *s = (const unsigned char *)src;
  unsigned char *d = (unsigned char *)dst;
  const size_t w = type_size(type);
  size_t rows = 1, width = 1;
  for (int a = 0; a < rank; ++a) {
    if ((axes_mask >> a) & 1u) width *= (size_t)dims[a];
    else rows *= (size_t)dims[a];
  }
  for (size_t r = 0; r < rows; ++r) {
    size_t remaining = r;
    int64_t base = 0;
    for (int a = rank - 1; a >= 0; --a) {
      if ((axes_mask >> a) & 1u) continue;
      base += (int64_t)(remaining % (size_t)dims[a]) * byte_strides[a];
      remaining /= (size_t)dims[a];
    }
    const int extremum = kind == HYLE_ORACLE_MIN || kind == HYLE_ORACLE_MAX;
    const int maximum = kind == HYLE_ORACLE_MAX;
    float result = extremum ? (maximum ? -INFINITY : INFINITY) : 0.0f;
    for (size_t c = 0; c < width; ++c) {
      remaining = c;
      int64_t offset = base;
      for (int a = rank - 1; a >= 0; --a) {
        if (!((axes_mask >> a) & 1u)) continue;
        offset += (int64_t)(remaining % (size_t)dims[a]) * byte_strides[a];
        remaining /= (size_t)dims[a];
      }
      const float value = load_as_f32(type, s + offset);
      if (extremum) accumulate_extremum(maximum, value, &result);
      else result += value;
    }
    if (kind == HYLE_ORACLE_MEAN) result = width == 0 ? NAN : result / (float)width;
    store_from_f32(type, d + r * w, result);
  }
}

/* include/hyle/simd/search.h:11-19 */
size_t hyle_oracle_index_of_max_f32(const float *data, size_t n) {
  if (n == 0) return 0;
  size_t best = 0;
  for (size_t i = 0; i < n; ++i) {
    if (isnan(data[i])) return i;
    if (data[i] > data[best]) best = i;
  }
  return best;
}

/* src/compute_provider_cuda/collectives.cu:478-495 (ArgBest, largest=true):
 * a NaN never beats a number; equal values (including -0 == +0) and NaN pairs
 * resolve to the lower index. */
void hyle_oracle_topk1_f32(const float *data, size_t rows, size_t width,
                           float *values, int32_t *indices) {
  for (size_t r = 0; r < rows; ++r) {
    const float *row = data + r * width;
    size_t best = 0;
    for (size_t i = 1; i < width; ++i) {
      const int best_nan = isnan(row[best]);
      const int cand_nan = isnan(row[i]);
      if (best_nan != cand_nan) {
        if (best_nan) best = i;
        continue;
      }
      if (!best_nan && row[i] > row[best]) best = i;
    }
    if (width != 0) {
      if (values) values[r] = row[best];
      if (indices) indices[r] = (int32_t)best;
    }
  }
}

/* TopK(count = k) along one axis of a plain strided tensor.  The order is the
 * reference's independent host ordering
 * (tests/compute_route_vulkan/topk_test_support.h:62-76): a stable sort in which
 * numbers precede NaNs, larger numbers come first (smaller when `largest` is 0),
 * and equal numbers (-0 == +0) as well as NaNs keep their index order.  Values
 * are copies of the source bits (include/hyle/compute/providers/cuda.h:113-116).
 * Outputs are dense with the axis extent replaced by k
 * (src/compute_ops/operation.cc:1622-1657). */
typedef struct {
  double value;  /* a float widened exactly, or an int32 */
  int32_t index;
} topk_item;
static int g_topk_largest;
static int topk_before(const void *pa, const void *pb) {
  const topk_item *a = (const topk_item *)pa, *b = (const topk_item *)pb;
  const int a_nan = isnan(a->value), b_nan = isnan(b->value);
  if (a_nan != b_nan) return a_nan ? 1 : -1;
  if (!a_nan && a->value != b->value) {
    const int a_first = g_topk_largest ? a->value > b->value : a->value < b->value;
    return a_first ? -1 : 1;
  }
  return a->index < b->index ? -1 : (a->index > b->index ? 1 : 0);
}
void hyle_oracle_topk(int type, const void *src, int rank, const int64_t *dims,
                      const int64_t *byte_strides, int axis, size_t k, int largest,
                      void *values, int32_t *indices) {
  const unsigned char *s = (const unsigned char *)src;
  unsigned char *v = (unsigned char *)values;
  const size_t w = type_size(type);
  const size_t width = (size_t)dims[axis];
  size_t outer = 1, inner = 1;
  for (int a = 0; a < axis; ++a) outer *= (size_t)dims[a];
  for (int a = axis + 1; a < rank; ++a) inner *= (size_t)dims[a];
  topk_item *items = (topk_item *)malloc((width ? width : 1) * sizeof(topk_item));
  g_topk_largest = largest;
  for (size_t row = 0; row < outer * inner; ++row) {
    size_t remaining = row;
    int64_t base = 0;
    for (int a = rank - 1; a >= 0; --a) {
      if (a == axis) continue;
      base += (int64_t)(remaining % (size_t)dims[a]) * byte_strides[a];
      remaining /= (size_t)dims[a];
    }
    for (size_t i = 0; i < width; ++i) {
      const unsigned char *at = s + base + (int64_t)i * byte_strides[axis];
      if (type == HYLE_ORACLE_I32) {
        int32_t whole;
        memcpy(&whole, at, sizeof whole);
        items[i].value = (double)whole;
      } else {
        items[i].value = (double)load_as_f32(type, at);
      }
      items[i].index = (int32_t)i;
    }
    qsort(items, width, sizeof(topk_item), topk_before);  /* a total order: index breaks ties */
    const size_t o = row / inner, lane = row % inner;
    for (size_t j = 0; j < k; ++j) {
      const size_t out = (o * k + j) * inner + lane;
      memcpy(v + out * w, s + base + (int64_t)items[j].index * byte_strides[axis], w);
      indices[out] = items[j].index;
    }
  }
  free(items);
}

/* ------------------------------------------------------------------------ */
/* Q8_0                                                                     */
/* ------------------------------------------------------------------------ */

/* Format constants: src/compute_ops/low_precision.cc:28-29 (32 elements, 34
 * bytes).  Decode restated from ggml dequantize_row_q8_0: y[j] = qs[j] * d
 * with d = fp16 -> f32.  |qs| <= 128 has at most 8 significant bits and d has
 * 11, so the f32 product is exact; the bf16 store is then a single RN-even. */
void hyle_oracle_q8_0_dequant_bf16(const void *blocks, size_t rows, size_t k,
                                   size_t row_stride_bytes, uint16_t *out,
                                   float *sumsq, float *sumsq_rounded) {
  const unsigned char *base = (const unsigned char *)blocks;
  const size_t nb = k / 32;
  for (size_t r = 0; r < rows; ++r) {
    const unsigned char *row = base + r * row_stride_bytes;
    float acc = 0.0f, acc_rounded = 0.0f;
    for (size_t b = 0; b < nb; ++b) {
      const unsigned char *blk = row + b * 34;
      const uint16_t dbits = (uint16_t)(blk[0] | ((uint16_t)blk[1] << 8));
      const float d = hyle_oracle_f16_to_f32(dbits);
      for (size_t j = 0; j < 32; ++j) {
        const float y = (float)(int8_t)blk[2 + j] * d;
        const uint16_t h = hyle_oracle_f32_to_bf16(y);
        out[r * k + b * 32 + j] = h;
        acc += y * y;
        const float yr = hyle_oracle_bf16_to_f32(h);
        acc_rounded += yr * yr;
      }
    }
    if (sumsq) sumsq[r] = acc;
    if (sumsq_rounded) sumsq_rounded[r] = acc_rounded;
  }
}

/* ------------------------------------------------------------------------ */
/* Q4_K, Q6_K                                                               */
/* ------------------------------------------------------------------------ */

/* Block geometry: src/compute_ops/low_precision.cc:22-27 (256 elements in 144
 * and 210 bytes).  The decode is ggml's (dequantize_row_q4_K / _q6_K, pinned
 * with the other GGUF formats at ffa4e8b... in cmake/HyleDependencyLock.json
 * and absent from the reference tree), restated from the published block
 * layouts:
 *   Q4_K  {f16 d; f16 dmin; u8 scales[12]; u8 qs[128]}: eight sub-blocks of 32
 *         with 6-bit scale sc and minimum m; y = (d * sc) * q - (dmin * m),
 *         q the low nibbles of qs[32 c .. 32 c + 31] for sub-block 2 c and the
 *         high nibbles for sub-block 2 c + 1;
 *   Q6_K  {u8 ql[128]; u8 qh[64]; i8 scales[16]; f16 d}: sixteen sub-blocks of
 *         16; y = (d * scale) * (q - 32), q six bits from ql (low four) and qh
 *         (high two).
 * Products and the subtraction are separate f32 roundings, as the source
 * writes them.  Pinned bit for bit against the two readings of these formats
 * the reference tree holds (third_party/ggml_q4k_apple/ggml_q4k_apple.h:9-38;
 * tests/compute_models/qwen27_original_nextn_reference.h:74-86,262-287). */
static void q4_k_scale_min(int j, const unsigned char *q, unsigned *scale, unsigned *minimum) {
  if (j < 4) {
    *scale = q[j] & 63u;
    *minimum = q[j + 4] & 63u;
  } else {
    *scale = (q[j + 4] & 0xFu) | ((unsigned)(q[j - 4] >> 6) << 4);
    *minimum = (unsigned)(q[j + 4] >> 4) | ((unsigned)(q[j] >> 6) << 4);
  }
}

static void q4_k_block_f32(const unsigned char *blk, float *y) {
  const float d = hyle_oracle_f16_to_f32((uint16_t)(blk[0] | ((uint16_t)blk[1] << 8)));
  const float dmin = hyle_oracle_f16_to_f32((uint16_t)(blk[2] | ((uint16_t)blk[3] << 8)));
  const unsigned char *scales = blk + 4, *q = blk + 16;
  for (int chunk = 0; chunk < 4; ++chunk) {
    unsigned sc, m;
    q4_k_scale_min(2 * chunk, scales, &sc, &m);
    const float d1 = d * (float)sc, m1 = dmin * (float)m;
    q4_k_scale_min(2 * chunk + 1, scales, &sc, &m);
    const float d2 = d * (float)sc, m2 = dmin * (float)m;
    for (int l = 0; l < 32; ++l) y[64 * chunk + l] = d1 * (float)(q[32 * chunk + l] & 0xF) - m1;
    for (int l = 0; l < 32; ++l) y[64 * chunk + 32 + l] = d2 * (float)(q[32 * chunk + l] >> 4) - m2;
  }
}

static void q6_k_block_f32(const unsigned char *blk, float *y) {
  const unsigned char *ql = blk, *qh = blk + 128;
  const int8_t *sc = (const int8_t *)(blk + 192);
  const float d = hyle_oracle_f16_to_f32((uint16_t)(blk[208] | ((uint16_t)blk[209] << 8)));
  for (int half = 0; half < 2; ++half) {
    for (int l = 0; l < 32; ++l) {
      const int is = l / 16;
      const int q1 = (int)((ql[l] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
      const int q2 = (int)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
      const int q3 = (int)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
      const int q4 = (int)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
      y[l] = d * (float)sc[is] * (float)q1;
      y[l + 32] = d * (float)sc[is + 2] * (float)q2;
      y[l + 64] = d * (float)sc[is + 4] * (float)q3;
      y[l + 96] = d * (float)sc[is + 6] * (float)q4;
    }
    y += 128;
    ql += 64;
    qh += 32;
    sc += 8;
  }
}

/* kind: 0 = Q4_K, 1 = Q6_K.  out_f32 and out_bf16 may each be NULL. */
void hyle_oracle_k_quant_dequant(int kind, const void *blocks, size_t rows, size_t k,
                                 size_t row_stride_bytes, float *out_f32, uint16_t *out_bf16,
                                 float *sumsq) {
  const unsigned char *base = (const unsigned char *)blocks;
  const size_t block_bytes = kind == 0 ? 144 : 210;
  float y[256];
  for (size_t r = 0; r < rows; ++r) {
    float acc = 0.0f;
    for (size_t b = 0; b < k / 256; ++b) {
      const unsigned char *blk = base + r * row_stride_bytes + b * block_bytes;
      if (kind == 0) q4_k_block_f32(blk, y);
      else q6_k_block_f32(blk, y);
      for (size_t j = 0; j < 256; ++j) {
        if (out_f32) out_f32[r * k + b * 256 + j] = y[j];
        if (out_bf16) out_bf16[r * k + b * 256 + j] = hyle_oracle_f32_to_bf16(y[j]);
        acc += y[j] * y[j];
      }
    }
    if (sumsq) sumsq[r] = acc;
  }
}

/* y[m][n] = sum_k w[n][k] * x[m][k] with w the exact f32 decode of a GGUF row
 * (kind 0 Q4_K, 1 Q6_K, 2 Q8_0) and double accumulation: the value the f32
 * kernel is held to within its summation-order bound.  `magnitude` (optional)
 * receives sum_k |w * x|, the scale of that bound.  This is MatMul with exact
 * weights; ggml's 8-bit activation quantisation is not restated. */
void hyle_oracle_gguf_matvec(int kind, const void *blocks, size_t rows, size_t k,
                             size_t row_stride_bytes, const float *x, size_t m,
                             double *out, double *magnitude) {
  const unsigned char *base = (const unsigned char *)blocks;
  float *w = (float *)malloc((k ? k : 1) * sizeof(float));
  if (w == NULL) return;
  for (size_t r = 0; r < rows; ++r) {
    const unsigned char *row = base + r * row_stride_bytes;
    if (kind == 2) {
      for (size_t b = 0; b < k / 32; ++b) {
        const unsigned char *blk = row + b * 34;
        const float d = hyle_oracle_f16_to_f32((uint16_t)(blk[0] | ((uint16_t)blk[1] << 8)));
        for (size_t j = 0; j < 32; ++j) w[b * 32 + j] = (float)(int8_t)blk[2 + j] * d;
      }
    } else {
      for (size_t b = 0; b < k / 256; ++b) {
        if (kind == 0) q4_k_block_f32(row + b * 144, w + b * 256);
        else q6_k_block_f32(row + b * 210, w + b * 256);
      }
    }
    for (size_t i = 0; i < m; ++i) {
      double sum = 0.0, size = 0.0;
      for (size_t j = 0; j < k; ++j) {
        const double term = (double)w[j] * (double)x[i * k + j];
        sum += term;
        size += fabs(term);
      }
      out[i * rows + r] = sum;
      if (magnitude) magnitude[i * rows + r] = size;
    }
  }
  free(w);
}

/* ------------------------------------------------------------------------ */
/* MatMul over a GGUF weight the way the reference's ggml CPU route computes  */
/* it: the activation row is quantised to 8-bit blocks first, block dot      */
/* products are integers, scales are applied in f32.  ggml's source is not    */
/* in the reference tree; the reference's tests restate its activation        */
/* codecs and the product they accept, and that restatement is followed here: */
/*   tests/compute_models/dspark_original_shared_reference.h:147-185 (Q8_0    */
/*     activation block, the AVX form), 219-262 (Q8_0 x Q8_0 centre + bound); */
/*   tests/compute_models/qwen27_original_nextn_reference.h:74-86 (scales,    */
/*     six-bit codes), 94-130 (weight groups), 144-167 (Q8_K activation       */
/*     block), 193-257 (centre + bound).                                      */
/* ------------------------------------------------------------------------ */
static float rn_divide(float a, float b) { return (float)((double)a / (double)b); }
static float rn_multiply(float a, float b) { return (float)((double)a * (double)b); }

/* Q8_0 activation blocks of 32: scale = f16(RN(max / 127)) widened again,
 * code = nearest-even integer of RN(x * RN(127 / max)). */
void hyle_oracle_quantize_q8_0(const float *x, size_t k, int8_t *codes, float *scales) {
  for (size_t b = 0; b < k / 32; ++b) {
    const float *v = x + 32 * b;
    float maximum = 0.0f;
    for (int i = 0; i < 32; ++i) maximum = fabsf(v[i]) > maximum ? fabsf(v[i]) : maximum;
    if (maximum == 0.0f) {
      scales[b] = 0.0f;
      memset(codes + 32 * b, 0, 32);
      continue;
    }
    const float divisor = rn_divide(maximum, 127.0f);
    scales[b] = hyle_oracle_f16_to_f32(hyle_oracle_f32_to_f16(divisor));
    const float reciprocal = rn_divide(127.0f, maximum);
    for (int i = 0; i < 32; ++i)
      codes[32 * b + i] = (int8_t)nearbyint((double)rn_multiply(v[i], reciprocal));
  }
}

/* Q8_K activation blocks of 256: the first element of largest magnitude, sign
 * kept, gives inverse = RN(-127 / max); code = min(127, nearest-even integer
 * of RN(x * inverse)); the stored f32 scale is RN(1 / inverse). */
void hyle_oracle_quantize_q8_k(const float *x, size_t k, int8_t *codes, float *scales) {
  for (size_t b = 0; b < k / 256; ++b) {
    const float *v = x + 256 * b;
    float maximum = 0.0f, absolute = 0.0f;
    for (int i = 0; i < 256; ++i)
      if (fabsf(v[i]) > absolute) {
        absolute = fabsf(v[i]);
        maximum = v[i];
      }
    if (absolute == 0.0f) {
      scales[b] = 0.0f;
      memset(codes + 256 * b, 0, 256);
      continue;
    }
    const float inverse = rn_divide(-127.0f, maximum);
    scales[b] = rn_divide(1.0f, inverse);
    for (int i = 0; i < 256; ++i) {
      const int code = (int)nearbyint((double)rn_multiply(v[i], inverse));
      codes[256 * b + i] = (int8_t)(code > 127 ? 127 : code);
    }
  }
}

typedef struct {
  double plain, correction;
} compensated_sum;
static void compensated_add(compensated_sum *s, double term) {
  const double next = s->plain + term;
  s->correction += fabs(s->plain) >= fabs(term) ? (s->plain - next) + term : (term - next) + s->plain;
  s->plain = next;
}
static double next_up(double v) { return nextafter(v, INFINITY); }
static double gamma_bound(size_t count, double unit) {
  const double product = (double)count * unit;
  return next_up(product / (1.0 - product));
}

/* One 32-wide group of a weight row: value_i = scale * codes[i] + minimum * offsets[i]. */
typedef struct {
  double scale, minimum;
  int codes[32], offsets[32];
} weight_group;

static weight_group gguf_weight_group(int kind, const unsigned char *row, size_t group) {
  weight_group g;
  memset(&g, 0, sizeof g);
  if (kind == 2) {
    const unsigned char *blk = row + group * 34;
    g.scale = hyle_oracle_f16_to_f32((uint16_t)(blk[0] | ((uint16_t)blk[1] << 8)));
    for (int i = 0; i < 32; ++i) g.codes[i] = (int8_t)blk[2 + i];
    return g;
  }
  const size_t local = group % 8;
  if (kind == 1) {
    const unsigned char *blk = row + (group / 8) * 210;
    g.scale = hyle_oracle_f16_to_f32((uint16_t)(blk[208] | ((uint16_t)blk[209] << 8)));
    for (int i = 0; i < 32; ++i) {
      const size_t column = local * 32 + (size_t)i;
      const size_t half = column / 128, within = column % 128, lane = within % 32, quarter = within / 32;
      const unsigned low = blk[half * 64 + lane + (quarter % 2) * 32], high = blk[128 + half * 32 + lane];
      const int code = (int)(((low >> (quarter >= 2 ? 4 : 0)) & 15u) | (((high >> (quarter * 2)) & 3u) << 4)) - 32;
      g.codes[i] = code * (int)(int8_t)blk[192 + column / 16];
    }
    return g;
  }
  const unsigned char *blk = row + (group / 8) * 144;
  g.scale = hyle_oracle_f16_to_f32((uint16_t)(blk[0] | ((uint16_t)blk[1] << 8)));
  g.minimum = hyle_oracle_f16_to_f32((uint16_t)(blk[2] | ((uint16_t)blk[3] << 8)));
  int scale, minimum;
  if (local < 4) {
    scale = blk[4 + local] & 63;
    minimum = blk[8 + local] & 63;
  } else {
    scale = (blk[8 + local] & 15) | ((blk[local] >> 6) << 4);
    minimum = (blk[8 + local] >> 4) | ((blk[4 + local] >> 6) << 4);
  }
  for (int i = 0; i < 32; ++i) {
    g.codes[i] = (int)((blk[16 + (local / 2) * 32 + i] >> (local % 2 ? 4 : 0)) & 15) * scale;
    g.offsets[i] = -minimum;
  }
  return g;
}

/* centre[i * rows + r]: the exact value of sum over groups of
 * w.scale * a.scale * (w.codes . a.codes) + w.minimum * a.scale * (w.offsets . a.codes)
 * (every term exact in double, compensated sum); bound[...]: the distance from
 * it the reference's test accepts of the native result,
 * gamma(k / 4 + 65, 2^-24) * sum |terms| plus the centre's own f64 error. */
void hyle_oracle_gguf_matvec_q8(int kind, const void *blocks, size_t rows, size_t k,
                                size_t row_stride_bytes, const float *x, size_t m,
                                double *centre, double *bound) {
  const size_t groups = k / 32;
  int8_t *codes = (int8_t *)malloc(k ? k : 1);
  float *scales = (float *)malloc((groups ? groups : 1) * sizeof(float));
  if (codes == NULL || scales == NULL) {
    free(codes);
    free(scales);
    return;
  }
  const double g32 = gamma_bound(k / 4 + 65, 0x1p-24), g64 = gamma_bound(2 * groups + 2, 0x1p-53);
  for (size_t i = 0; i < m; ++i) {
    if (kind == 2) {
      hyle_oracle_quantize_q8_0(x + i * k, k, codes, scales);
    } else {  /* one f32 scale per 256: spread over the eight groups it covers */
      hyle_oracle_quantize_q8_k(x + i * k, k, codes, scales);
      for (size_t g = groups; g-- > 0;) scales[g] = scales[g / 8];
    }
    for (size_t r = 0; r < rows; ++r) {
      const unsigned char *row = (const unsigned char *)blocks + r * row_stride_bytes;
      compensated_sum sum = {0.0, 0.0};
      double absolute = 0.0;
      for (size_t g = 0; g < groups; ++g) {
        const weight_group w = gguf_weight_group(kind, row, g);
        const double a_scale = scales[g];
        const int8_t *a = codes + 32 * g;
        for (int part = 0; part < 2; ++part) {
          const double scale = part == 0 ? w.scale : w.minimum;
          const int *c = part == 0 ? w.codes : w.offsets;
          if (scale == 0.0) continue;
          long dot = 0, size = 0;
          for (int j = 0; j < 32; ++j) {
            dot += (long)c[j] * a[j];
            size += labs((long)c[j]) * labs((long)a[j]);
          }
          compensated_add(&sum, scale * a_scale * (double)dot);
          absolute = next_up(absolute + next_up(fabs(scale) * next_up(fabs(a_scale) * (double)size)));
        }
      }
      const double value = sum.plain + sum.correction;
      centre[i * rows + r] = value;
      if (bound) {
        const double own = next_up(next_up(fabs(value - sum.plain)) + next_up(g64 * absolute));
        bound[i * rows + r] = next_up(next_up(g32 * absolute) + own);
      }
    }
  }
  free(codes);
  free(scales);
}

void hyle_oracle_q8_0_dequant_f32(const void *blocks, size_t rows, size_t k,
                                  size_t row_stride_bytes, float *out) {
  const unsigned char *base = (const unsigned char *)blocks;
  const size_t nb = k / 32;
  for (size_t r = 0; r < rows; ++r) {
    const unsigned char *row = base + r * row_stride_bytes;
    for (size_t b = 0; b < nb; ++b) {
      const unsigned char *blk = row + b * 34;
      const uint16_t dbits = (uint16_t)(blk[0] | ((uint16_t)blk[1] << 8));
      const float d = hyle_oracle_f16_to_f32(dbits);
      for (size_t j = 0; j < 32; ++j)
        out[r * k + b * 32 + j] = (float)(int8_t)blk[2 + j] * d;
    }
  }
}

/* ------------------------------------------------------------------------ */
/* Cast / Copy                                                              */
/* ------------------------------------------------------------------------ */

/* src/compute_provider_native/cast.cc:19-41: nearest-even IEEE binary32 of an
 * int32, formed from the integer so it does not depend on the ambient rounding
 * mode. */
static float int32_to_float32(int32_t value) {
  const uint32_t raw = (uint32_t)value;
  const uint32_t sign = raw & 0x80000000u;
  const uint32_t magnitude = value < 0 ? 0u - raw : raw;
  if (magnitude == 0) return 0.0f;
  unsigned exponent = 31u - (unsigned)__builtin_clz(magnitude);
  uint32_t significand;
  if (exponent <= 23) {
    significand = magnitude << (23 - exponent);
  } else {
    const unsigned shift = exponent - 23;
    significand = magnitude >> shift;
    const uint32_t remainder = magnitude & ((1u << shift) - 1);
    const uint32_t halfway = 1u << (shift - 1);
    if (remainder > halfway || (remainder == halfway && (significand & 1u)))
      ++significand;
    if (significand == (1u << 24)) {
      significand >>= 1;
      ++exponent;
    }
  }
  const uint32_t bits = sign | ((exponent + 127) << 23) | (significand & 0x7FFFFFu);
  float out;
  memcpy(&out, &bits, 4);
  return out;
}

static size_t cast_type_size(int type) {
  switch (type) {
    case HYLE_ORACLE_F32:
    case HYLE_ORACLE_I32: return 4;
    case HYLE_ORACLE_F16:
    case HYLE_ORACLE_BF16: return 2;
    case HYLE_ORACLE_BOOL: return 1;
    default: return 0;
  }
}

static int is_float_type(int type) {
  return type == HYLE_ORACLE_F32 || type == HYLE_ORACLE_F16 || type == HYLE_ORACLE_BF16;
}

/* src/compute_provider_native/cast.cc:73-92 (convert_value) and 225-238 (the
 * strided walk); same type: src/compute_provider_native/transform.cc:85-89
 * (bytes are kept). */
int hyle_oracle_cast(int src_type, int dst_type, const void *src,
                     const int64_t *dims, const int64_t *strides, int rank,
                     void *dst) {
  const size_t sw = cast_type_size(src_type), dw = cast_type_size(dst_type);
  if (sw == 0 || dw == 0) return -1;
  const int same = src_type == dst_type;
  if (!same) {
    const int ok = (is_float_type(src_type) && is_float_type(dst_type)) ||
                   (src_type == HYLE_ORACLE_I32 && dst_type == HYLE_ORACLE_F32) ||
                   (src_type == HYLE_ORACLE_BOOL && is_float_type(dst_type)) ||
                   (is_float_type(src_type) && dst_type == HYLE_ORACLE_BOOL);
    if (!ok) return -1;
  }
  const size_t n = element_count(dims, rank);
  const unsigned char *s = (const unsigned char *)src;
  unsigned char *d = (unsigned char *)dst;
  for (size_t i = 0; i < n; ++i) {
    const unsigned char *from =
        s + hyle_oracle_logical_byte_offset(dims, strides, rank, i);
    unsigned char *to = d + i * dw;
    if (same) {
      memcpy(to, from, sw);
    } else if (src_type == HYLE_ORACLE_I32) {
      int32_t v;
      memcpy(&v, from, 4);
      const float f = int32_to_float32(v);
      memcpy(to, &f, 4);
    } else if (dst_type == HYLE_ORACLE_BOOL) {
      /* truth of the stored bits: any nonzero magnitude, subnormals and NaNs
       * included; both zeros are false */
      uint32_t bits = 0;
      memcpy(&bits, from, sw);
      const uint32_t magnitude = sw == 4 ? 0x7FFFFFFFu : 0x7FFFu;
      *to = (unsigned char)((bits & magnitude) != 0);
    } else if (src_type == HYLE_ORACLE_BOOL) {
      store_from_f32(dst_type, to, *from != 0 ? 1.0f : 0.0f);
    } else {
      store_from_f32(dst_type, to, load_as_f32(src_type, from));
    }
  }
  return 0;
}

/* src/compute_provider_cuda/tensor_kernel.cu:190-193: every element takes the
 * scalar's bits (ScalarValue::bits, include/hyle/compute/operation.h:187-230). */
void hyle_oracle_fill(size_t width, uint64_t bits, size_t n, void *dst) {
  unsigned char *d = (unsigned char *)dst;
  for (size_t i = 0; i < n; ++i)
    for (size_t b = 0; b < width; ++b)
      d[i * width + b] = (unsigned char)(bits >> (8 * b));
}

/* src/compute_provider_cuda/tensor_kernel.cu:194-198 with the operand offsets of
 * tensor_provider.cc:176-189 (an operand axis of extent 1, or one the operand
 * lacks, contributes nothing): the condition byte picks the branch, whose
 * `width` bytes are kept as they are. */
void hyle_oracle_select(size_t width, const void *condition,
                        const int64_t *condition_dims, const int64_t *condition_strides, int condition_rank,
                        const void *first, const int64_t *first_dims, const int64_t *first_strides, int first_rank,
                        const void *second, const int64_t *second_dims, const int64_t *second_strides, int second_rank,
                        const int64_t *out_dims, int out_rank, void *dst) {
  const size_t n = element_count(out_dims, out_rank);
  unsigned char *d = (unsigned char *)dst;
  for (size_t i = 0; i < n; ++i) {
    const unsigned char mask = ((const unsigned char *)condition)[hyle_oracle_broadcast_byte_offset(
        condition_dims, condition_strides, condition_rank, out_dims, out_rank, i)];
    const unsigned char *from =
        mask != 0 ? (const unsigned char *)first + hyle_oracle_broadcast_byte_offset(
                                                      first_dims, first_strides, first_rank, out_dims, out_rank, i)
                  : (const unsigned char *)second + hyle_oracle_broadcast_byte_offset(
                                                       second_dims, second_strides, second_rank, out_dims, out_rank, i);
    memcpy(d + i * width, from, width);
  }
}

/* src/compute_ops/operation.cc:1516-1564 (shape) and the storage rule of
 * include/hyle/compute/providers/cuda.h:38-43: input `i` (dims equal to the
 * output's except on `axis`, any byte strides) lands at `offset` on the axis of
 * the dense output, its `width`-byte elements kept as they are.  One call per
 * input. */
void hyle_oracle_concat_part(size_t width, const void *src, const int64_t *dims,
                             const int64_t *strides, int rank, int axis, int64_t offset,
                             const int64_t *out_dims, void *dst) {
  const size_t n = element_count(dims, rank);
  unsigned char *d = (unsigned char *)dst;
  for (size_t i = 0; i < n; ++i) {
    size_t rest = i, to = 0, scale = 1;
    for (int a = rank - 1; a >= 0; --a) {
      const size_t c = rest % (size_t)dims[a];
      rest /= (size_t)dims[a];
      to += (a == axis ? c + (size_t)offset : c) * scale;
      scale *= (size_t)out_dims[a];
    }
    memcpy(d + to * width,
           (const unsigned char *)src + hyle_oracle_logical_byte_offset(dims, strides, rank, i), width);
  }
}

/* ---- Gather -------------------------------------------------------------- */
/* src/compute_provider_native/indexing.cc:57-91,143-276: the output is the
 * source with `axis` replaced by the shape of the indices; output element at
 * coordinates (before, item.., after) is the source element at (before,
 * indices[item..], after), `width` bytes kept as they are.  Checked bounds look
 * at every index first: one below 0 or at / past the axis extent returns 1 and
 * writes nothing (indexing.cc:75-91), as does an axis of extent 0 under either
 * policy (indexing.cc:189-195). */
static int64_t read_gather_index(const unsigned char *indices, int wide, size_t offset) {
  if (wide) {
    int64_t value;
    memcpy(&value, indices + offset, sizeof value);
    return value;
  }
  int32_t value;
  memcpy(&value, indices + offset, sizeof value);
  return value;
}

int hyle_oracle_gather(size_t width, const void *src, const int64_t *dims, const int64_t *strides, int rank,
                       int axis, const void *indices, int wide, const int64_t *index_dims,
                       const int64_t *index_strides, int index_rank, int checked, void *dst) {
  int64_t out_dims[16];
  int out_rank = 0;
  for (int a = 0; a < axis; ++a) out_dims[out_rank++] = dims[a];
  for (int a = 0; a < index_rank; ++a) out_dims[out_rank++] = index_dims[a];
  for (int a = axis + 1; a < rank; ++a) out_dims[out_rank++] = dims[a];
  const size_t n = element_count(out_dims, out_rank);
  if (n == 0) return 0;
  if (dims[axis] == 0) return 1;
  const size_t index_count = element_count(index_dims, index_rank);
  const unsigned char *ids = (const unsigned char *)indices;
  if (checked) {
    for (size_t i = 0; i < index_count; ++i) {
      const int64_t value =
          read_gather_index(ids, wide, hyle_oracle_logical_byte_offset(index_dims, index_strides, index_rank, i));
      if (value < 0 || (uint64_t)value >= (uint64_t)dims[axis]) return 1;
    }
  }
  unsigned char *d = (unsigned char *)dst;
  for (size_t i = 0; i < n; ++i) {
    size_t coordinate[16];
    size_t rest = i;
    for (int a = out_rank - 1; a >= 0; --a) {
      coordinate[a] = rest % (size_t)out_dims[a];
      rest /= (size_t)out_dims[a];
    }
    size_t index_offset = 0;
    for (int a = 0; a < index_rank; ++a) index_offset += coordinate[axis + a] * (size_t)index_strides[a];
    const int64_t selected = read_gather_index(ids, wide, index_offset);
    size_t from = 0;
    for (int a = 0; a < rank; ++a) {
      const size_t c = a < axis ? coordinate[a] : a == axis ? (size_t)selected : coordinate[a - 1 + index_rank];
      from += c * (size_t)strides[a];
    }
    memcpy(d + i * width, (const unsigned char *)src + from, width);
  }
  return 0;
}

/* ---- RoPE ---------------------------------------------------------------- */
/* src/compute_ggml_runtime/explicit_rope.h:11-74: data widened to f32, positions
 * converted to f32, phase = frequency * position in f32, cosf / sinf of the
 * phase, a' = a * cos - b * sin and b' = a * sin + b * cos with every product
 * and sum a separate f32 operation, one rounding to the storage type; elements
 * past `rotary` are copied.  Pairs: (2i, 2i + 1) interleaved, (i, i + rotary / 2)
 * half-split.  Positions are [S] or (batched) the data's leading dimensions
 * through the sequence axis; frequencies [rotary / 2] or (stepped) [S, rotary / 2]. */
void hyle_oracle_rope(int type, const void *data, const int64_t *dims, int rank, int sequence_axis,
                      const void *positions, int wide, int batched, const float *frequencies, int stepped,
                      int64_t rotary, int half_split, void *dst) {
  const size_t depth = (size_t)dims[rank - 1], pairs = (size_t)rotary / 2;
  const size_t n = element_count(dims, rank);
  if (n == 0) return;
  const size_t rows = n / depth, sequence = (size_t)dims[sequence_axis];
  size_t inner = 1;
  for (int a = sequence_axis + 1; a < rank - 1; ++a) inner *= (size_t)dims[a];
  const size_t size = type_size(type);
  const unsigned char *src = (const unsigned char *)data;
  unsigned char *out = (unsigned char *)dst;
  for (size_t r = 0; r < rows; ++r) {
    const size_t step_index = r / inner, step = step_index % sequence;
    const size_t at = batched ? step_index : step;
    const float position = wide ? (float)((const int64_t *)positions)[at] : (float)((const int32_t *)positions)[at];
    const float *row_frequencies = frequencies + (stepped ? step * pairs : 0);
    const size_t base = r * depth;
    for (size_t i = 0; i < pairs; ++i) {
      const size_t first = base + (half_split ? i : 2 * i), second = half_split ? first + pairs : first + 1;
      const volatile float phase = row_frequencies[i] * position;
      const float c = cosf(phase), sn = sinf(phase);
      const float a = load_as_f32(type, src + first * size), b = load_as_f32(type, src + second * size);
      const volatile float ac = a * c, bs = b * sn, as = a * sn, bc = b * c;
      store_from_f32(type, out + first * size, ac - bs);
      store_from_f32(type, out + second * size, as + bc);
    }
    for (size_t i = (size_t)rotary; i < depth; ++i) memcpy(out + (base + i) * size, src + (base + i) * size, size);
  }
}

/* ---- Sampling ------------------------------------------------------------ */
/* Philox4x32-10 as the reference addresses it (third_party/random123_counter/
 * philox.h:20-44; include/hyle/compute/sampling_ops.h:12-16): identity = key
 * low / high, draw low / high; block `index` is the counter {index low, index
 * high, draw low, draw high} under that key. */
void hyle_oracle_philox_block(const uint32_t identity[4], uint64_t index, uint32_t out[4]) {
  uint32_t x0 = (uint32_t)index, x1 = (uint32_t)(index >> 32), x2 = identity[2], x3 = identity[3];
  uint32_t key0 = identity[0], key1 = identity[1];
  for (int round = 0; round < 10; ++round) {
    const uint64_t first = (uint64_t)0xD2511F53u * x0;
    const uint64_t second = (uint64_t)0xCD9E8D57u * x2;
    const uint32_t y0 = (uint32_t)(second >> 32) ^ x1 ^ key0;
    const uint32_t y2 = (uint32_t)(first >> 32) ^ x3 ^ key1;
    x1 = (uint32_t)second;
    x3 = (uint32_t)first;
    x0 = y0;
    x2 = y2;
    key0 += 0x9E3779B9u;
    key1 += 0xBB67AE85u;
  }
  out[0] = x0, out[1] = x1, out[2] = x2, out[3] = x3;
}

/* RandomBits (src/compute_provider_native/sampling.cc:77-88): word j of row r
 * is lane j % 4 of block j / 4 under the row's identity. */
void hyle_oracle_random_bits(const uint32_t *identities, size_t rows, size_t word_count, uint32_t *out) {
  for (size_t r = 0; r < rows; ++r)
    for (size_t column = 0; column < word_count; column += 4) {
      uint32_t words[4];
      hyle_oracle_philox_block(identities + 4 * r, column / 4, words);
      for (size_t lane = 0; lane < 4 && column + lane < word_count; ++lane) out[r * word_count + column + lane] = words[lane];
    }
}

/* The uniform of a row's draw (sampling.cc:155-158): the 52-bit midpoint of the
 * first two words of block 0, in (0, 1). */
double hyle_oracle_categorical_uniform(const uint32_t identity[4]) {
  uint32_t words[4];
  hyle_oracle_philox_block(identity, 0, words);
  return ((double)words[0] * 0x1p20 + (double)(words[1] >> 12) + 0.5) * 0x1p-52;
}

/* Categorical (sampling.cc:119-182,184-215): per row the maximum, the mass
 * total = sum of expf(x - max) in double, and the first index whose running
 * mass exceeds total * uniform; a threshold that rounding leaves past the last
 * boundary selects the last element equal to the maximum.  The optional score
 * is (x[selected] - max) - log(total) in double, narrowed.  NaN, +Inf or a row
 * without finite elements returns 1 and writes nothing. */
static void load_row_f32(int type, const void *base, size_t first, size_t count, float *dst) {
  const unsigned char *bytes = (const unsigned char *)base + first * type_size(type);
  for (size_t i = 0; i < count; ++i) dst[i] = load_as_f32(type, bytes + i * type_size(type));
}

int hyle_oracle_categorical(int type, const void *logits, const uint32_t *identities, size_t rows, size_t width,
                            int32_t *indices, float *log_probabilities) {
  float *row = (float *)malloc((width ? width : 1) * sizeof(float));
  float *maxima = (float *)malloc((rows ? rows : 1) * sizeof(float));
  int invalid = 0;
  for (size_t r = 0; r < rows; ++r) {
    load_row_f32(type, logits, r * width, width, row);
    float maximum = -INFINITY;
    for (size_t c = 0; c < width; ++c) {
      if (isnan(row[c]) || row[c] == INFINITY) invalid = 1;
      maximum = row[c] > maximum ? row[c] : maximum;
    }
    if (!isfinite(maximum)) invalid = 1;
    maxima[r] = maximum;
  }
  for (size_t r = 0; r < rows && !invalid; ++r) {
    load_row_f32(type, logits, r * width, width, row);
    const float maximum = maxima[r];
    double total = 0;
    for (size_t c = 0; c < width; ++c) total += (double)expf(row[c] - maximum);
    const double threshold = total * hyle_oracle_categorical_uniform(identities + 4 * r);
    double cumulative = 0;
    size_t selected = width;
    for (size_t c = 0; c < width; ++c) {
      cumulative += (double)expf(row[c] - maximum);
      if (cumulative > threshold) {
        selected = c;
        break;
      }
    }
    if (selected == width)
      for (selected = width; selected > 0; --selected)
        if (row[selected - 1] == maximum) {
          --selected;
          break;
        }
    indices[r] = (int32_t)selected;
    if (log_probabilities != NULL)
      log_probabilities[r] = (float)((double)row[selected] - (double)maximum - log(total));
  }
  free(row);
  free(maxima);
  return invalid;
}

/* ------------------------------------------------------------------------ */
/* CPU baseline legs (row ranges, dense loops)                              */
/* ------------------------------------------------------------------------ */

void hyle_oracle_rows_add_row_scale_f32(const float *a, const float *b, float s,
                                        float *out, size_t cols,
                                        size_t row_begin, size_t row_end) {
  for (size_t r = row_begin; r < row_end; ++r) {
    const float *row = a + r * cols;
    float *dst = out + r * cols;
    for (size_t c = 0; c < cols; ++c) dst[c] = row[c] + b[c];
    for (size_t c = 0; c < cols; ++c) dst[c] = dst[c] * s;
  }
}

void hyle_oracle_rows_add_bf16(const uint16_t *r, const uint16_t *y,
                               uint16_t *out, size_t cols, size_t row_begin,
                               size_t row_end) {
  float left[128], right[128];
  for (size_t row = row_begin; row < row_end; ++row) {
    for (size_t c = 0; c < cols; c += 128) {
      const size_t size = cols - c < 128 ? cols - c : 128;
      const size_t base = row * cols + c;
      for (size_t i = 0; i < size; ++i) left[i] = hyle_oracle_bf16_to_f32(r[base + i]);
      for (size_t i = 0; i < size; ++i) right[i] = hyle_oracle_bf16_to_f32(y[base + i]);
      for (size_t i = 0; i < size; ++i) left[i] = left[i] + right[i];
      for (size_t i = 0; i < size; ++i) out[base + i] = hyle_oracle_f32_to_bf16(left[i]);
    }
  }
}

void hyle_oracle_rows_swiglu_bf16(const uint16_t *gate, const uint16_t *up,
                                  uint16_t *out, size_t cols, size_t row_begin,
                                  size_t row_end) {
  float g[128], u[128];
  for (size_t row = row_begin; row < row_end; ++row) {
    for (size_t c = 0; c < cols; c += 128) {
      const size_t size = cols - c < 128 ? cols - c : 128;
      const size_t base = row * cols + c;
      for (size_t i = 0; i < size; ++i) g[i] = hyle_oracle_bf16_to_f32(gate[base + i]);
      for (size_t i = 0; i < size; ++i) u[i] = hyle_oracle_bf16_to_f32(up[base + i]);
      for (size_t i = 0; i < size; ++i) g[i] = hyle_oracle_silu(g[i]) * u[i];
      for (size_t i = 0; i < size; ++i) out[base + i] = hyle_oracle_f32_to_bf16(g[i]);
    }
  }
}

void hyle_oracle_rows_rms_norm_bf16(const uint16_t *x, const uint16_t *w,
                                    uint16_t *out, size_t cols, float epsilon,
                                    size_t row_begin, size_t row_end) {
  hyle_oracle_rms_norm_native(HYLE_ORACLE_BF16, HYLE_ORACLE_BF16,
                              x + row_begin * cols, w, out + row_begin * cols,
                              row_end - row_begin, cols, epsilon);
}

void hyle_oracle_rows_softmax_bool_f32(const float *x, const uint8_t *mask,
                                       float *out, size_t cols,
                                       size_t mask_rows, size_t row_begin,
                                       size_t row_end) {
  for (size_t r = row_begin; r < row_end; ++r) {
    const float *src = x + r * cols;
    const uint8_t *m = mask + (r % mask_rows) * cols;
    float *dst = out + r * cols;
    for (size_t c = 0; c < cols; ++c) dst[c] = m[c] ? src[c] : -INFINITY;
    hyle_oracle_softmax_f32_row(dst, dst, cols);
  }
}

void hyle_oracle_rows_topk1_f32(const float *x, float *values, int32_t *indices,
                                size_t cols, size_t row_begin, size_t row_end) {
  hyle_oracle_topk1_f32(x + row_begin * cols, row_end - row_begin, cols,
                        values + row_begin, indices + row_begin);
}

void hyle_oracle_rows_q8_0_bf16(const void *blocks, uint16_t *out, float *sumsq,
                                size_t k, size_t row_stride, size_t row_begin,
                                size_t row_end) {
  hyle_oracle_q8_0_dequant_bf16((const unsigned char *)blocks + row_begin * row_stride,
                                row_end - row_begin, k, row_stride,
                                out + row_begin * k, sumsq + row_begin, NULL);
}
