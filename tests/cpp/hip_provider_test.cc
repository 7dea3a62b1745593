// Tests of the C++ host mirror (include/hyle_hip_compute.hpp) in the shape of the reference's
// provider tests (tests/compute_provider_native/elementwise_test.cc, normalization_test.cc,
// transformer_test.cc, reduction_test.cc; tests/compute_provider_cuda/native_reduction_test.cc):
// describe -> prepare -> create_invocation -> submit -> wait -> compare.
//
//   hip_provider_test --host     schema, inference, admission and error behaviour; no device used
//   hip_provider_test --device   the same calls executed on device 0, compared with the CPU oracle
//
// The oracle (oracle/hyle_oracle.h) is linked here as the checker only.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <functional>
#include <limits>
#include <random>
#include <string>
#include <vector>

#include "hyle_hip_compute.hpp"
#include "hyle_oracle.h"

namespace {

using namespace hyle::compute;
using hyle::Status;

struct Case { const char *name; bool device; std::function<void()> body; };
std::vector<Case> &cases() { static std::vector<Case> all; return all; }
int failures = 0;

struct Registrar {
  Registrar(const char *name, bool device, std::function<void()> body) { cases().push_back({name, device, std::move(body)}); }
};
#define HOST_TEST(name) void name(); Registrar reg_##name(#name, false, name); void name()
#define DEVICE_TEST(name) void name(); Registrar reg_##name(#name, true, name); void name()
#define EXPECT(cond) do { if (!(cond)) { ++failures; std::printf("  FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); } } while (0)
#define REQUIRE(cond) do { if (!(cond)) { ++failures; std::printf("  FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); return; } } while (0)

constexpr float kInf = std::numeric_limits<float>::infinity();
constexpr float kNaN = std::numeric_limits<float>::quiet_NaN();

TensorDesc dense(DataType type, std::initializer_list<std::int64_t> dims) { return TensorDesc::dense(type, dims).value(); }

// ---------------------------------------------------------------- host ----------------------------
HOST_TEST(TensorDescDenseStridesAndZeroExtents) {
  const TensorDesc d = dense(DataType::kBFloat16, {4, 3, 8});
  EXPECT(d.rank() == 3 && d.is_dense());
  EXPECT(d.byte_strides()[0] == 48 && d.byte_strides()[1] == 16 && d.byte_strides()[2] == 2);
  EXPECT(d.element_count() == 96 && d.required_bytes() == 192);
  const TensorDesc empty = dense(DataType::kFloat32, {4, 0, 8});
  EXPECT(empty.is_dense() && empty.required_bytes() == 0);
  EXPECT(empty.byte_strides()[0] == 0 && empty.byte_strides()[2] == 0);
  EXPECT(TensorDesc::dense(DataType::kFloat32, {2, -1}).error().IsInvalidArgument());
  const auto broadcast = TensorDesc::strided_bytes(DataType::kFloat32, {4, 8}, {0, 4});
  REQUIRE(broadcast.has_value());
  EXPECT(!broadcast->is_dense() && broadcast->required_bytes() == 32);
  const auto q8 = TensorDesc::gguf_q8_0_weight(DataType::kBFloat16, 2048, 16);
  REQUIRE(q8.has_value());
  EXPECT(!q8->is_plain() && q8->required_bytes() == 16 * 64 * 34);
  EXPECT(TensorDesc::gguf_q8_0_weight(DataType::kBFloat16, 2040, 16).error().IsInvalidArgument());
}

HOST_TEST(InfersOutputsLikeTheSchema) {
  auto out = infer_output_descriptions(Binary{BinaryKind::kAdd},
                                       {dense(DataType::kFloat32, {6, 1, 5}), dense(DataType::kFloat32, {4, 5})});
  REQUIRE(out.has_value() && out->size() == 1);
  EXPECT((*out)[0] == dense(DataType::kFloat32, {6, 4, 5}));
  EXPECT(infer_output_descriptions(Binary{}, {dense(DataType::kFloat32, {3}), dense(DataType::kFloat32, {4})})
             .error().IsInvalidArgument());
  EXPECT(infer_output_descriptions(Binary{}, {dense(DataType::kFloat32, {3}), dense(DataType::kBFloat16, {3})})
             .error().IsInvalidArgument());
  out = infer_output_descriptions(TopK{}, {dense(DataType::kFloat32, {7, 100})});
  REQUIRE(out.has_value() && out->size() == 2);
  EXPECT((*out)[0] == dense(DataType::kFloat32, {7, 1}) && (*out)[1] == dense(DataType::kInt32, {7, 1}));
  out = infer_output_descriptions(GatedActivation{}, {dense(DataType::kBFloat16, {9, 64})});
  REQUIRE(out.has_value());
  EXPECT((*out)[0] == dense(DataType::kBFloat16, {9, 32}));
  EXPECT(infer_output_descriptions(GatedActivation{}, {dense(DataType::kBFloat16, {9, 63})}).error().IsInvalidArgument());
  out = infer_output_descriptions(Reduce{ReductionKind::kMaximum, *Axes::from(std::array<std::int32_t, 1>{-1}), true}, {dense(DataType::kFloat32, {3, 9})});
  REQUIRE(out.has_value());
  EXPECT((*out)[0] == dense(DataType::kFloat32, {3, 1}));
  out = infer_output_descriptions(Q8_0DequantSumSquares{}, {*TensorDesc::gguf_weight(TensorDesc::GgufQuantizedType::kQ6K, DataType::kBFloat16, 512, 3)});
  REQUIRE(out.has_value() && out->size() == 2);
  EXPECT((*out)[0] == dense(DataType::kBFloat16, {3, 512}) && (*out)[1] == dense(DataType::kFloat32, {3}));
  EXPECT(TensorDesc::gguf_weight(TensorDesc::GgufQuantizedType::kQ4K, DataType::kBFloat16, 300, 3).error().IsInvalidArgument());
  out = infer_output_descriptions(GgufMatVec{}, {*TensorDesc::gguf_weight(TensorDesc::GgufQuantizedType::kQ4K, DataType::kBFloat16, 512, 7),
                                                 dense(DataType::kFloat32, {3, 512})});
  REQUIRE(out.has_value() && out->size() == 1);
  EXPECT((*out)[0] == dense(DataType::kFloat32, {3, 7}));
  EXPECT(infer_output_descriptions(GgufMatVec{}, {*TensorDesc::gguf_weight(TensorDesc::GgufQuantizedType::kQ4K, DataType::kBFloat16, 512, 7),
                                                  dense(DataType::kFloat32, {3, 256})}).error().IsInvalidArgument());
  out = infer_output_descriptions(Q8_0DequantSumSquares{}, {*TensorDesc::gguf_q8_0_weight(DataType::kBFloat16, 64, 5)});
  REQUIRE(out.has_value() && out->size() == 2);
  EXPECT((*out)[0] == dense(DataType::kBFloat16, {5, 64}) && (*out)[1] == dense(DataType::kFloat32, {5}));
  EXPECT(infer_output_descriptions(RmsNorm{}, {dense(DataType::kBFloat16, {4, 64}), dense(DataType::kBFloat16, {32})})
             .error().IsInvalidArgument());
  EXPECT(infer_output_descriptions(Softmax{.axis = 2}, {dense(DataType::kFloat32, {4, 64})}).error().IsOutOfRange() ||
         infer_output_descriptions(Softmax{.axis = 2}, {dense(DataType::kFloat32, {4, 64})}).error().IsInvalidArgument());
}

HOST_TEST(PreparesRoutesAndDeclinesCleanly) {
  const Context context = Context::planning_only();
  auto add = prepare(context, Binary{BinaryKind::kAdd}, dense(DataType::kFloat32, {32, 256}), dense(DataType::kFloat32, {256}));
  REQUIRE(add.has_value());
  EXPECT(add->dispatch_count() == 1 && add->workspace_requirement().size == 0);
  EXPECT(add->alias_support(0, 0)->supported && !add->alias_support(0, 1)->supported);
  EXPECT(*add->output_description() == dense(DataType::kFloat32, {32, 256}));
  auto top = prepare(context, TopK{}, dense(DataType::kFloat32, {8, 151936}));
  REQUIRE(top.has_value());
  EXPECT(top->dispatch_count() == 2 && top->workspace_requirement().size > 0);
  EXPECT(top->create_invocation().error().IsInvalidArgument());  // needs its workspace
  // Declines are Unimplemented, never an error a router would have to surface.
  auto top4 = prepare(context, TopK{.count = 4}, dense(DataType::kFloat32, {8, 128}));
  REQUIRE(top4.has_value());
  EXPECT(std::string(top4->route_name()) == "topk-select-tiles" && top4->workspace_requirement().size == 0);
  EXPECT(prepare(context, TopK{.count = 1025}, dense(DataType::kFloat32, {8, 4096})).has_value());
  EXPECT(prepare(context, TopK{.count = 3}, dense(DataType::kInt32, {8, 4096})).has_value());
  EXPECT(prepare(context, TopK{.count = 3}, dense(DataType::kUInt8, {8, 4096})).error().IsUnimplemented());
  auto folded = prepare(context, Reduce{ReductionKind::kSum, *Axes::from(std::array<std::int32_t, 2>{0, 2})},
                        dense(DataType::kFloat32, {4, 5, 6}));
  REQUIRE(folded.has_value());
  EXPECT(std::string(folded->route_name()) == "reduce-strided");
  EXPECT(prepare(context, Unary{UnaryKind::kAbs}, dense(DataType::kInt32, {8})).error().IsUnimplemented());
  EXPECT(prepare(context, LayerNorm{1.0e-5F, DataType::kFloat16}, dense(DataType::kFloat16, {8, 64})).error().IsUnimplemented());
  EXPECT(prepare(context, Unary{UnaryKind::kTanh}, dense(DataType::kFloat32, {8})).has_value());
  EXPECT(prepare(context, GatedActivation{GatedActivationKind::kGelu}, dense(DataType::kBFloat16, {8, 64})).has_value());
  EXPECT(prepare(context, Binary{}, dense(DataType::kInt32, {8}), dense(DataType::kInt32, {8})).error().IsUnimplemented());
  // Schema violations stay InvalidArgument.
  EXPECT(prepare(context, Binary{}, dense(DataType::kFloat32, {3}), dense(DataType::kFloat32, {4})).error().IsInvalidArgument());
  // Zero elements: prepared, nothing to dispatch.
  auto none = prepare(context, Binary{}, dense(DataType::kFloat32, {0, 8}), dense(DataType::kFloat32, {8}));
  REQUIRE(none.has_value());
  EXPECT(none->dispatch_count() == 0);
}

HOST_TEST(CastAndCopyInferDenseOutputsAndDeclineUndefinedPairs) {
  const Context context = Context::planning_only();
  const TensorDesc strided = *TensorDesc::strided_bytes(DataType::kFloat16, {2, 2}, {5, 2});
  auto out = infer_output_descriptions(Cast{DataType::kFloat32}, {strided});
  REQUIRE(out.has_value());
  EXPECT((*out)[0] == dense(DataType::kFloat32, {2, 2}));
  out = infer_output_descriptions(Copy{}, {strided});
  REQUIRE(out.has_value());
  EXPECT((*out)[0] == dense(DataType::kFloat16, {2, 2}));
  EXPECT(infer_output_descriptions(Cast{}, {dense(DataType::kFloat32, {4})}).error().IsInvalidArgument());
  auto narrow = prepare(context, Cast{DataType::kBFloat16}, dense(DataType::kFloat32, {8192, 2048}));
  REQUIRE(narrow.has_value());
  EXPECT(narrow->dispatch_count() == 1 && !narrow->alias_support(0, 0)->supported);
  // tests/compute_provider_native/cast_test.cc:296-301: the reverse integer pair is not defined
  EXPECT(prepare(context, Cast{DataType::kInt32}, dense(DataType::kFloat32, {2, 8})).error().IsUnimplemented());
  EXPECT(prepare(context, Cast{DataType::kFloat32}, dense(DataType::kInt32, {2, 8})).has_value());
}

HOST_TEST(FillAndSelectFollowTheSchema) {
  const Context context = Context::planning_only();
  // src/compute_ops/operation.cc:1263-1275
  auto out = infer_output_descriptions(Fill{{3, 5}, DataType::kFloat32, ScalarValue(1.0F)}, {});
  REQUIRE(out.has_value());
  EXPECT((*out)[0] == dense(DataType::kFloat32, {3, 5}));
  EXPECT(infer_output_descriptions(Fill{{3}, DataType::kBFloat16, ScalarValue(1.0F)}, {}).error().IsInvalidArgument());
  EXPECT(infer_output_descriptions(Fill{{3}, DataType::kUnknown, ScalarValue()}, {}).error().IsInvalidArgument());
  auto filled = prepare(context, Fill{{8192, 2048}, DataType::kBFloat16, ScalarValue::from_bits(DataType::kBFloat16, 0x3F80)});
  REQUIRE(filled.has_value());
  EXPECT(filled->dispatch_count() == 1);
  // src/compute_ops/operation.cc:1309-1330
  out = infer_output_descriptions(Select{}, {dense(DataType::kBool, {4, 1, 6}), dense(DataType::kInt8, {5, 6}),
                                             dense(DataType::kInt8, {4, 5, 1})});
  REQUIRE(out.has_value());
  EXPECT((*out)[0] == dense(DataType::kInt8, {4, 5, 6}));
  EXPECT(infer_output_descriptions(Select{}, {dense(DataType::kUInt8, {8}), dense(DataType::kFloat32, {8}),
                                              dense(DataType::kFloat32, {8})}).error().IsInvalidArgument());
  EXPECT(infer_output_descriptions(Select{}, {dense(DataType::kBool, {8}), dense(DataType::kFloat32, {8}),
                                              dense(DataType::kFloat16, {8})}).error().IsInvalidArgument());
  auto selected = prepare(context, Select{}, dense(DataType::kBool, {8, 16}), dense(DataType::kFloat32, {8, 16}),
                          dense(DataType::kFloat32, {}));
  REQUIRE(selected.has_value());
  EXPECT(!selected->alias_support(0, 0)->supported && selected->alias_support(0, 1)->supported &&
         !selected->alias_support(0, 2)->supported);
}

HOST_TEST(ConcatFollowsTheSchema) {
  const Context context = Context::planning_only();
  // src/compute_ops/operation.cc:1516-1564: equal types and extents off the axis, negative axes count from the end
  auto out = infer_output_descriptions(Concat{-1}, {dense(DataType::kFloat16, {2, 3, 5}), dense(DataType::kFloat16, {2, 3, 0}),
                                                    dense(DataType::kFloat16, {2, 3, 7})});
  REQUIRE(out.has_value());
  EXPECT((*out)[0] == dense(DataType::kFloat16, {2, 3, 12}));
  EXPECT(infer_output_descriptions(Concat{0}, {dense(DataType::kFloat16, {2, 3}), dense(DataType::kFloat32, {2, 3})}).error().IsInvalidArgument());
  EXPECT(infer_output_descriptions(Concat{0}, {dense(DataType::kFloat16, {2, 3}), dense(DataType::kFloat16, {2, 4})}).error().IsInvalidArgument());
  EXPECT(infer_output_descriptions(Concat{2}, {dense(DataType::kFloat16, {2, 3})}).error().IsOutOfRange());  // operation.cc:228-242
  // a group of a wider Concat: the output keeps its whole extent, the group says where it starts
  out = infer_output_descriptions(Concat{1, 20, 9}, {dense(DataType::kInt32, {4, 3}), dense(DataType::kInt32, {4, 5})});
  REQUIRE(out.has_value());
  EXPECT((*out)[0] == dense(DataType::kInt32, {4, 20}));
  EXPECT(infer_output_descriptions(Concat{1, 20, 15}, {dense(DataType::kInt32, {4, 3}), dense(DataType::kInt32, {4, 5})}).error().IsInvalidArgument());
  auto prepared = prepare(context, Concat{1}, dense(DataType::kBFloat16, {8192, 2048}), dense(DataType::kBFloat16, {8192, 4096}));
  REQUIRE(prepared.has_value());
  EXPECT(prepared->dispatch_count() == 1);
  EXPECT(!prepared->alias_support(0, 0)->supported && !prepared->alias_support(0, 1)->supported);
}

HOST_TEST(GatherFollowsTheSchema) {
  const Context context = Context::planning_only();
  // src/compute_ops/operation.cc:616-637,1470-1489
  auto out = infer_output_descriptions(Gather{1}, {dense(DataType::kFloat64, {2, 7, 3}), dense(DataType::kInt64, {2, 3})});
  REQUIRE(out.has_value());
  EXPECT((*out)[0] == dense(DataType::kFloat64, {2, 2, 3, 3}));
  EXPECT(infer_output_descriptions(Gather{0}, {dense(DataType::kFloat32, {4, 3}), dense(DataType::kFloat32, {2})}).error().IsInvalidArgument());
  EXPECT(infer_output_descriptions(Gather{2}, {dense(DataType::kFloat32, {4, 3}), dense(DataType::kInt32, {2})}).error().IsOutOfRange());
  auto checked = prepare(context, Gather{0}, dense(DataType::kBFloat16, {151936, 2048}), dense(DataType::kInt32, {8192}));
  REQUIRE(checked.has_value());
  // large enough to check inside the moving blocks: one dispatch; 20000 indices take the checking dispatch first
  EXPECT(checked->dispatch_count() == 1 && checked->workspace_requirement().size != 0);
  auto many = prepare(context, Gather{0}, dense(DataType::kBFloat16, {151936, 2048}), dense(DataType::kInt32, {20000}));
  REQUIRE(many.has_value());
  EXPECT(many->dispatch_count() == 2 && many->workspace_requirement().size == checked->workspace_requirement().size);
  auto trusted = prepare(context, Gather{0, IndexBoundsPolicy::kUnchecked}, dense(DataType::kBFloat16, {151936, 2048}),
                         dense(DataType::kInt32, {8192}));
  REQUIRE(trusted.has_value());
  EXPECT(trusted->dispatch_count() == 1 && trusted->workspace_requirement().size == 0);
}

HOST_TEST(SubmitWithoutDeviceIsFailedPrecondition) {
  Context context = Context::planning_only();
  EXPECT(context.create_queue().error().IsFailedPrecondition());
}

// -------------------------------------------------------------- device ----------------------------
struct Fixture {
  Context context = Context::create(hip::device(0)).value();
  Queue queue = context.create_queue().value();
};
Fixture &fixture() { static Fixture f; return f; }

template <class T> DeviceBuffer upload(const std::vector<T> &host) {
  DeviceBuffer b = DeviceBuffer::create(host.size() * sizeof(T)).value();
  EXPECT(b.write(host.data(), host.size() * sizeof(T)).ok());
  return b;
}
template <class T> std::vector<T> download(const DeviceBuffer &b, std::size_t count) {
  std::vector<T> host(count);
  EXPECT(b.read(host.data(), count * sizeof(T)).ok());
  return host;
}
std::vector<float> normal(std::size_t n, unsigned seed, float sigma = 1.0F) {
  std::mt19937 rng(seed);
  std::normal_distribution<float> dist(0.0F, sigma);
  std::vector<float> v(n);
  for (float &x : v) x = dist(rng);
  return v;
}
std::vector<std::uint16_t> to_bf16(const std::vector<float> &v) {
  std::vector<std::uint16_t> r(v.size());
  hyle_oracle_convert_from_f32(HYLE_ORACLE_BF16, v.data(), r.data(), v.size());
  return r;
}
bool same_bits(const void *a, const void *b, std::size_t bytes) { return std::memcmp(a, b, bytes) == 0; }
// bf16 results may differ from the oracle by one unit in the last place (fused vs. scalar order).
bool within_one_ulp_bf16(const std::vector<std::uint16_t> &got, const std::vector<std::uint16_t> &want) {
  for (std::size_t i = 0; i < got.size(); ++i) {
    const auto key = [](std::uint16_t b) { return (b & 0x8000U) ? -static_cast<int>(b & 0x7FFFU) : static_cast<int>(b & 0x7FFFU); };
    const bool nan_g = (got[i] & 0x7FFFU) > 0x7F80U, nan_w = (want[i] & 0x7FFFU) > 0x7F80U;
    if (nan_g != nan_w) return false;
    if (!nan_g && std::abs(key(got[i]) - key(want[i])) > 1) return false;
  }
  return true;
}

DEVICE_TEST(BinaryAddBroadcastsRowVectorBitExactly) {
  constexpr std::int64_t rows = 37, cols = 1000;  // not a multiple of the vector width
  const auto a = normal(rows * cols, 1), b = normal(cols, 2);
  const TensorDesc da = dense(DataType::kFloat32, {rows, cols}), db = dense(DataType::kFloat32, {cols});
  auto prepared = prepare(fixture().context, Binary{BinaryKind::kAdd}, da, db);
  REQUIRE(prepared.has_value());
  DeviceBuffer left = upload(a), right = upload(b), out = DeviceBuffer::create(a.size() * 4).value();
  auto invocation = prepared->create_invocation();
  REQUIRE(invocation.has_value());
  auto completion = invocation->submit(fixture().queue, *ConstTensorView::create(da, left), *ConstTensorView::create(db, right),
                                       *TensorView::create(da, out));
  REQUIRE(completion.has_value());
  EXPECT(completion->wait().ok());
  std::vector<float> want(a.size());
  const std::int64_t ad[2] = {rows, cols}, as[2] = {cols * 4, 4}, bd[1] = {cols}, bs[1] = {4};
  hyle_oracle_binary(HYLE_ORACLE_ADD, HYLE_ORACLE_F32, a.data(), ad, as, 2, b.data(), bd, bs, 1, want.data(), ad, 2);
  EXPECT(same_bits(download<float>(out, a.size()).data(), want.data(), a.size() * 4));
  // In place over the left operand, which the plan reports as supported.
  EXPECT(prepared->alias_support(0, 0)->supported);
  completion = invocation->submit(fixture().queue, *ConstTensorView::create(da, left), *ConstTensorView::create(db, right),
                                  *TensorView::create(da, left));
  REQUIRE(completion.has_value());
  EXPECT(completion->wait().ok());
  EXPECT(same_bits(download<float>(left, a.size()).data(), want.data(), a.size() * 4));
}

DEVICE_TEST(BinaryChainEqualsTwoBinaries) {
  constexpr std::int64_t rows = 64, cols = 512;
  const auto a = normal(rows * cols, 3), b = normal(cols, 4);
  const std::vector<float> s{0.125F};
  const TensorDesc da = dense(DataType::kFloat32, {rows, cols}), db = dense(DataType::kFloat32, {cols}),
                   ds = dense(DataType::kFloat32, {});
  auto prepared = prepare(fixture().context, BinaryChain{BinaryKind::kAdd, BinaryKind::kMultiply}, da, db, ds);
  REQUIRE(prepared.has_value());
  DeviceBuffer ba = upload(a), bb = upload(b), bs = upload(s), out = DeviceBuffer::create(a.size() * 4).value();
  auto invocation = prepared->create_invocation().value();
  auto completion = invocation.submit(fixture().queue,
                                      {*ConstTensorView::create(da, ba), *ConstTensorView::create(db, bb), *ConstTensorView::create(ds, bs)},
                                      {*TensorView::create(da, out)});
  REQUIRE(completion.has_value());
  EXPECT(completion->wait().ok());
  const auto got = download<float>(out, a.size());
  bool same = true;
  for (std::int64_t r = 0; r < rows && same; ++r)
    for (std::int64_t c = 0; c < cols; ++c) {
      const float want = (a[r * cols + c] + b[c]) * s[0];
      same = same && same_bits(&want, &got[r * cols + c], 4);
    }
  EXPECT(same);
}

DEVICE_TEST(RmsNormBf16WithinOneUlpOfScalarFloor) {
  constexpr std::int64_t rows = 33, hidden = 2048;
  const auto x = to_bf16(normal(rows * hidden, 5, 2.0F)), w = to_bf16(normal(hidden, 6));
  const TensorDesc dx = dense(DataType::kBFloat16, {rows, hidden}), dw = dense(DataType::kBFloat16, {hidden});
  auto prepared = prepare(fixture().context, RmsNorm{1.0e-6F}, dx, dw);
  REQUIRE(prepared.has_value());
  DeviceBuffer bx = upload(x), bw = upload(w), out = DeviceBuffer::create(x.size() * 2).value();
  auto completion = prepared->create_invocation()->submit(fixture().queue, *ConstTensorView::create(dx, bx),
                                                          *ConstTensorView::create(dw, bw), *TensorView::create(dx, out));
  REQUIRE(completion.has_value());
  EXPECT(completion->wait().ok());
  std::vector<std::uint16_t> want(x.size());
  hyle_oracle_rms_norm(HYLE_ORACLE_BF16, HYLE_ORACLE_BF16, x.data(), w.data(), want.data(), rows, hidden, 1.0e-6F);
  EXPECT(within_one_ulp_bf16(download<std::uint16_t>(out, x.size()), want));
}

DEVICE_TEST(SwigluSeparateBf16WithinOneUlp) {
  constexpr std::int64_t rows = 17, width = 6144;
  auto g = normal(rows * width, 7, 3.0F);
  g[0] = -kInf; g[1] = kInf; g[2] = kNaN; g[3] = -0.0F; g[4] = -100.0F;
  const auto gate = to_bf16(g), up = to_bf16(normal(rows * width, 8));
  const TensorDesc d = dense(DataType::kBFloat16, {rows, width});
  auto prepared = prepare(fixture().context, GatedActivation{GatedActivationKind::kSilu, GatedInputKind::kSeparate}, d, d);
  REQUIRE(prepared.has_value());
  DeviceBuffer bg = upload(gate), bu = upload(up), out = DeviceBuffer::create(gate.size() * 2).value();
  auto completion = prepared->create_invocation()->submit(fixture().queue, *ConstTensorView::create(d, bg),
                                                          *ConstTensorView::create(d, bu), *TensorView::create(d, out));
  REQUIRE(completion.has_value());
  EXPECT(completion->wait().ok());
  std::vector<std::uint16_t> want(gate.size());
  hyle_oracle_swiglu(HYLE_ORACLE_BF16, gate.data(), up.data(), want.data(), gate.size());
  EXPECT(within_one_ulp_bf16(download<std::uint16_t>(out, gate.size()), want));
}

DEVICE_TEST(SoftmaxBooleanMaskAndInvalidRows) {
  constexpr std::int64_t heads = 3, seq = 192;
  auto x = normal(heads * seq * seq, 9, 4.0F);
  std::vector<std::uint8_t> mask(seq * seq);
  for (std::int64_t q = 0; q < seq; ++q)
    for (std::int64_t k = 0; k < seq; ++k) mask[q * seq + k] = k <= q;
  for (std::int64_t k = 0; k < seq; ++k) mask[5 * seq + k] = 0;  // a fully masked row -> NaN row
  x[(seq + 7) * seq + 3] = kNaN;                                   // head 1, row 7 holds a NaN -> NaN row
  const TensorDesc dx = dense(DataType::kFloat32, {heads, seq, seq}), dm = dense(DataType::kBool, {seq, seq});
  auto prepared = prepare(fixture().context, Softmax{.mask = MaskKind::kBoolean}, dx, dm);
  REQUIRE(prepared.has_value());
  DeviceBuffer bx = upload(x), bm = upload(mask), out = DeviceBuffer::create(x.size() * 4).value();
  auto completion = prepared->create_invocation()->submit(fixture().queue, *ConstTensorView::create(dx, bx),
                                                          *ConstTensorView::create(dm, bm), *TensorView::create(dx, out));
  REQUIRE(completion.has_value());
  EXPECT(completion->wait().ok());
  std::vector<float> want(x.size());
  const std::int64_t xd[3] = {heads, seq, seq}, md[2] = {seq, seq}, ms[2] = {seq, 1};
  hyle_oracle_softmax(HYLE_ORACLE_F32, x.data(), want.data(), xd, 3, 1.0F, HYLE_ORACLE_MASK_BOOLEAN, mask.data(), md, ms, 2);
  const auto got = download<float>(out, x.size());
  bool close = true;
  for (std::size_t i = 0; i < got.size() && close; ++i) {
    if (std::isnan(want[i])) close = std::isnan(got[i]);
    else close = std::fabs(got[i] - want[i]) <= 1.0e-5F * std::fabs(want[i]) + 1.0e-9F;  // 1e-5 relative
  }
  EXPECT(close);
  EXPECT(std::isnan(got[5 * seq]) && std::isnan(got[(seq + 7) * seq]) && got[0] == 1.0F);
}

DEVICE_TEST(TopKArgmaxOrdersNaNLastAndTiesLow) {
  constexpr std::int64_t rows = 6, width = 151936;
  auto x = normal(rows * width, 10);
  x[0 * width + 777] = 9.0F; x[0 * width + 140000] = 9.0F;      // tie -> lower index
  x[1 * width + 5] = kNaN; x[1 * width + 90000] = 8.0F;          // NaN never wins over a number
  for (std::int64_t i = 0; i < width; ++i) x[2 * width + i] = kNaN;  // all NaN -> index 0
  for (std::int64_t i = 0; i < width; ++i) x[3 * width + i] = -kInf;
  x[3 * width + width - 1] = -1.0e30F;
  x[4 * width + 100] = kInf;
  const TensorDesc dx = dense(DataType::kFloat32, {rows, width});
  auto prepared = prepare(fixture().context, TopK{}, dx);
  REQUIRE(prepared.has_value());
  const WorkspaceRequirement need = prepared->workspace_requirement();
  DeviceBuffer bx = upload(x), values = DeviceBuffer::create(rows * 4).value(), indices = DeviceBuffer::create(rows * 4).value(),
               workspace = DeviceBuffer::create(need.size).value();
  auto invocation = prepared->create_invocation(workspace.data(), workspace.size());
  REQUIRE(invocation.has_value());
  auto completion = invocation->submit(fixture().queue, {*ConstTensorView::create(dx, bx)},
                                       {*TensorView::create(*prepared->output_description(0), values),
                                        *TensorView::create(*prepared->output_description(1), indices)});
  REQUIRE(completion.has_value());
  EXPECT(completion->wait().ok());
  std::vector<float> want_values(rows);
  std::vector<std::int32_t> want_indices(rows);
  hyle_oracle_topk1_f32(x.data(), rows, width, want_values.data(), want_indices.data());
  const auto got_indices = download<std::int32_t>(indices, rows);
  EXPECT(got_indices == want_indices);
  EXPECT(same_bits(download<float>(values, rows).data(), want_values.data(), rows * 4));
  EXPECT(got_indices[0] == 777 && got_indices[1] == 90000 && got_indices[2] == 0 && got_indices[3] == width - 1 && got_indices[4] == 100);
}

DEVICE_TEST(Q8_0DequantBitExactWithRowSumSquares) {
  constexpr std::int64_t n = 96, k = 2048, blocks = k / 32;
  std::mt19937 rng(11);
  std::vector<std::uint8_t> weight(n * blocks * 34);
  for (std::int64_t b = 0; b < n * blocks; ++b) {
    const std::uint16_t d = hyle_oracle_f32_to_f16(std::ldexp(static_cast<float>(rng() % 2048) / 2048.0F + 0.5F, -static_cast<int>(rng() % 12)));
    std::memcpy(&weight[b * 34], &d, 2);
    for (int j = 0; j < 32; ++j) weight[b * 34 + 2 + j] = static_cast<std::uint8_t>(rng());
  }
  const TensorDesc dw = *TensorDesc::gguf_q8_0_weight(DataType::kBFloat16, k, n);
  auto prepared = prepare(fixture().context, Q8_0DequantSumSquares{}, dw);
  REQUIRE(prepared.has_value());
  DeviceBuffer bw = upload(weight), out = DeviceBuffer::create(n * k * 2).value(), sumsq = DeviceBuffer::create(n * 4).value();
  auto completion = prepared->create_invocation()->submit(fixture().queue, {*ConstTensorView::create(dw, bw)},
                                                          {*TensorView::create(*prepared->output_description(0), out),
                                                           *TensorView::create(*prepared->output_description(1), sumsq)});
  REQUIRE(completion.has_value());
  EXPECT(completion->wait().ok());
  std::vector<std::uint16_t> want(n * k);
  std::vector<float> want_sumsq(n);
  hyle_oracle_q8_0_dequant_bf16(weight.data(), n, k, blocks * 34, want.data(), want_sumsq.data(), nullptr);
  EXPECT(same_bits(download<std::uint16_t>(out, n * k).data(), want.data(), n * k * 2));
  const auto got_sumsq = download<float>(sumsq, n);
  bool close = true;
  for (std::int64_t r = 0; r < n; ++r) close = close && std::fabs(got_sumsq[r] - want_sumsq[r]) <= 1.0e-5F * want_sumsq[r];
  EXPECT(close);  // summation order differs from the index-order oracle: 1e-5 relative
}

// MatMul over a GGUF weight as the reference's ggml CPU route computes it, on one of the reference's own
// projection widths (1024: tests/compute_models/cpu_c5_gguf_inputs.h:231), held to the bound its tests
// accept of that route (tests/compute_models/dspark_original_shared_reference.h:219-262).
DEVICE_TEST(GgufMatMulInTheGgmlRouteArithmeticOverAReferenceWidth) {
  constexpr std::int64_t n = 200, k = 1024, blocks = k / 32, m = 3;
  std::mt19937 rng(21);
  std::vector<std::uint8_t> weight(n * blocks * 34);
  for (std::int64_t b = 0; b < n * blocks; ++b) {
    const std::uint16_t d = hyle_oracle_f32_to_f16(std::ldexp(static_cast<float>(rng() % 2048) / 2048.0F + 0.5F, -static_cast<int>(4 + rng() % 8)));
    std::memcpy(&weight[b * 34], &d, 2);
    for (int j = 0; j < 32; ++j) weight[b * 34 + 2 + j] = static_cast<std::uint8_t>(rng());
  }
  const std::vector<float> x = normal(m * k, 22, 1.5F);
  const TensorDesc dw = *TensorDesc::gguf_q8_0_weight(DataType::kFloat32, k, n);
  const TensorDesc dx = *TensorDesc::dense(DataType::kFloat32, {m, k});
  auto prepared = prepare(fixture().context, GgufMatVec{ActivationArithmetic::kGgmlQ8}, dw, dx);
  REQUIRE(prepared.has_value());
  DeviceBuffer bw = upload(weight), bx = upload(x), out = DeviceBuffer::create(m * n * 4).value();
  auto completion = prepared->create_invocation()->submit(fixture().queue,
                                                          {*ConstTensorView::create(dw, bw), *ConstTensorView::create(dx, bx)},
                                                          {*TensorView::create(*prepared->output_description(0), out)});
  REQUIRE(completion.has_value());
  EXPECT(completion->wait().ok());
  EXPECT(std::string(hyle_hip_last_launch_variant()) == "gguf_matvec_q8_blocks/q8_0/4-tokens");
  std::vector<double> centre(m * n), bound(m * n);
  hyle_oracle_gguf_matvec_q8(2, weight.data(), n, k, blocks * 34, x.data(), m, centre.data(), bound.data());
  const auto got = download<float>(out, m * n);
  bool inside = true;
  for (std::int64_t i = 0; i < m * n; ++i) inside = inside && std::fabs(static_cast<double>(got[i]) - centre[i]) <= bound[i];
  EXPECT(inside);
}

DEVICE_TEST(CastNarrowsWidensAndMaterialisesStridedInputBitExactly) {
  constexpr std::int64_t rows = 257, cols = 2048;
  auto values = normal(rows * cols, 12, 2.0F);
  values[0] = kNaN; values[1] = kInf; values[2] = -0.0F; values[3] = 1.0e-40F; values[4] = 3.4e38F;
  const TensorDesc wide = dense(DataType::kFloat32, {rows, cols}), narrow = dense(DataType::kBFloat16, {rows, cols});
  auto prepared = prepare(fixture().context, Cast{DataType::kBFloat16}, wide);
  REQUIRE(prepared.has_value());
  DeviceBuffer source = upload(values), target = DeviceBuffer::create(values.size() * 2).value();
  auto completion = prepared->create_invocation()->submit(fixture().queue, *ConstTensorView::create(wide, source),
                                                          *TensorView::create(narrow, target));
  REQUIRE(completion.has_value());
  EXPECT(completion->wait().ok());
  std::vector<std::uint16_t> want(values.size());
  const std::int64_t dims[2] = {rows, cols}, wide_strides[2] = {cols * 4, 4}, narrow_strides[2] = {cols * 2, 2};
  EXPECT(hyle_oracle_cast(HYLE_ORACLE_F32, HYLE_ORACLE_BF16, values.data(), dims, wide_strides, 2, want.data()) == 0);
  const auto got = download<std::uint16_t>(target, values.size());
  EXPECT(same_bits(got.data(), want.data(), want.size() * 2));
  // and back: bf16 -> f32 is exact
  auto widen = prepare(fixture().context, Cast{DataType::kFloat32}, narrow);
  REQUIRE(widen.has_value());
  DeviceBuffer back = DeviceBuffer::create(values.size() * 4).value();
  completion = widen->create_invocation()->submit(fixture().queue, *ConstTensorView::create(narrow, target),
                                                  *TensorView::create(wide, back));
  REQUIRE(completion.has_value());
  EXPECT(completion->wait().ok());
  std::vector<float> widened(values.size());
  EXPECT(hyle_oracle_cast(HYLE_ORACLE_BF16, HYLE_ORACLE_F32, want.data(), dims, narrow_strides, 2, widened.data()) == 0);
  EXPECT(same_bits(download<float>(back, values.size()).data(), widened.data(), widened.size() * 4));
  // tests/compute_provider_native/cast_test.cc:177-183: f16 [2,2] with byte strides {5,2}
  std::vector<std::uint8_t> physical(16, 0);
  const std::uint16_t halves[4] = {0x3C00, 0x4000, 0x4200, 0x4400};
  const std::size_t offsets[4] = {0, 2, 5, 7};
  for (int i = 0; i < 4; ++i) std::memcpy(&physical[offsets[i]], &halves[i], 2);
  const TensorDesc strided = *TensorDesc::strided_bytes(DataType::kFloat16, {2, 2}, {5, 2});
  auto gather = prepare(fixture().context, Cast{DataType::kFloat32}, strided);
  REQUIRE(gather.has_value());
  DeviceBuffer raw = upload(physical), four = DeviceBuffer::create(16).value();
  completion = gather->create_invocation()->submit(fixture().queue, *ConstTensorView::create(strided, raw),
                                                   *TensorView::create(dense(DataType::kFloat32, {2, 2}), four));
  REQUIRE(completion.has_value());
  EXPECT(completion->wait().ok());
  EXPECT((download<float>(four, 4) == std::vector<float>{1.0F, 2.0F, 3.0F, 4.0F}));
  // Cast takes no alias: output over the input is refused
  EXPECT(prepared->create_invocation()->submit(fixture().queue, *ConstTensorView::create(wide, source),
                                               *TensorView::create(narrow, source)).error().IsInvalidArgument());
}

DEVICE_TEST(FillThenSelectKeepsBitsLikeTheReferenceRouteTest) {
  // tests/compute_route_vulkan/tensor_test.cc:255-283: alternating flags, a NaN-payload scalar,
  // Select(mask, input, filled) keeps the input's bits where the flag is set
  constexpr std::int64_t count = 4099;
  constexpr std::uint32_t scalar = 0xFFC00003U;
  std::vector<std::uint32_t> raw(count);
  std::mt19937 rng(7);
  for (auto &word : raw) word = rng();
  std::vector<std::uint8_t> flags(count);
  for (std::int64_t i = 0; i < count; ++i) flags[i] = static_cast<std::uint8_t>(i % 2);
  const TensorDesc values = dense(DataType::kFloat32, {count}), mask = dense(DataType::kBool, {count});
  auto fill = prepare(fixture().context, Fill{{count}, DataType::kFloat32, ScalarValue::from_bits(DataType::kFloat32, scalar)});
  REQUIRE(fill.has_value());
  DeviceBuffer filled = DeviceBuffer::create(count * 4).value();
  auto fill_invocation = fill->create_invocation();
  REQUIRE(fill_invocation.has_value());
  auto completion = fill_invocation->submit(fixture().queue, *TensorView::create(values, filled));
  REQUIRE(completion.has_value());
  EXPECT(completion->wait().ok());
  EXPECT(download<std::uint32_t>(filled, count) == std::vector<std::uint32_t>(count, scalar));
  auto select = prepare(fixture().context, Select{}, mask, values, values);
  REQUIRE(select.has_value());
  DeviceBuffer condition = upload(flags), input = upload(raw), out = DeviceBuffer::create(count * 4).value();
  auto invocation = select->create_invocation();
  REQUIRE(invocation.has_value());
  completion = invocation->submit(fixture().queue, *ConstTensorView::create(mask, condition), *ConstTensorView::create(values, input),
                                  *ConstTensorView::create(values, filled), *TensorView::create(values, out));
  REQUIRE(completion.has_value());
  EXPECT(completion->wait().ok());
  std::vector<std::uint32_t> want(count);
  const std::int64_t dims[1] = {count}, byte_stride[1] = {1}, word_stride[1] = {4};
  const std::vector<std::uint32_t> fill_words(count, scalar);
  hyle_oracle_select(4, flags.data(), dims, byte_stride, 1, raw.data(), dims, word_stride, 1, fill_words.data(), dims,
                     word_stride, 1, dims, 1, want.data());
  for (std::int64_t i = 0; i < count; ++i) EXPECT(want[i] == (flags[i] ? raw[i] : scalar));
  EXPECT(download<std::uint32_t>(out, count) == want);
}

DEVICE_TEST(ConcatJoinsRawWordsAlongTheMiddleAxis) {
  // tests/compute_route_vulkan/concat_test.cc:9-70: base [2, 3, 5], parts of 3, 0 and 4 along axis 1
  const std::int64_t extents[3] = {3, 0, 4}, out_dims[3] = {2, 7, 5};
  const TensorDesc joined = dense(DataType::kFloat32, {2, 7, 5});
  std::mt19937 rng(11);
  std::vector<std::vector<std::uint32_t>> parts;
  std::vector<DeviceBuffer> buffers;
  std::vector<TensorDesc> descs;
  std::vector<std::uint32_t> want(2 * 7 * 5, 0);
  std::int64_t offset = 0;
  for (std::int64_t extent : extents) {
    std::vector<std::uint32_t> words(2 * extent * 5);
    for (auto &word : words) word = rng();
    const std::int64_t dims[3] = {2, extent, 5}, strides[3] = {extent * 20, 20, 4};
    hyle_oracle_concat_part(4, words.data(), dims, strides, 3, 1, offset, out_dims, want.data());
    offset += extent;
    descs.push_back(dense(DataType::kFloat32, {2, extent, 5}));
    buffers.push_back(words.empty() ? DeviceBuffer::create(4).value() : upload(words));
    parts.push_back(std::move(words));
  }
  auto concat = prepare(fixture().context, Concat{1}, descs[0], descs[1], descs[2]);
  REQUIRE(concat.has_value());
  DeviceBuffer out = DeviceBuffer::create(want.size() * 4).value();
  auto invocation = concat->create_invocation();
  REQUIRE(invocation.has_value());
  auto completion = invocation->submit(fixture().queue, *ConstTensorView::create(descs[0], buffers[0]),
                                       *ConstTensorView::create(descs[1], buffers[1]), *ConstTensorView::create(descs[2], buffers[2]),
                                       *TensorView::create(joined, out));
  REQUIRE(completion.has_value());
  EXPECT(completion->wait().ok());
  for (std::int64_t i = 0; i < 2; ++i)
    for (std::int64_t j = 0; j < 7; ++j)
      for (std::int64_t k = 0; k < 5; ++k)
        EXPECT(want[(i * 7 + j) * 5 + k] == (j < 3 ? parts[0][(i * 3 + j) * 5 + k] : parts[2][(i * 4 + j - 3) * 5 + k]));
  EXPECT(download<std::uint32_t>(out, want.size()) == want);
}

DEVICE_TEST(CheckedGatherFailsTheCompletionAndKeepsTheOutput) {
  // tests/compute_provider_cuda/gather_collectives_test.cc:172-212: [4, 3] source, two Int64 indices;
  // -1, the extent, the largest and the smallest index fail with OutOfRange and write nothing
  const TensorDesc source = dense(DataType::kFloat64, {4, 3}), indices = dense(DataType::kInt64, {2});
  const std::vector<std::uint64_t> data{1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12}, poison{8, 7, 6, 5, 4, 3};
  auto gather = prepare(fixture().context, Gather{}, source, indices);
  REQUIRE(gather.has_value());
  const TensorDesc result = gather->output_description().value();
  EXPECT(result == dense(DataType::kFloat64, {2, 3}));
  DeviceBuffer input = upload(data);
  DeviceBuffer scratch = DeviceBuffer::create(gather->workspace_requirement().size).value();
  const std::int64_t dims[2] = {4, 3}, strides[2] = {24, 8}, index_dims[1] = {2}, index_strides[1] = {8};
  for (std::int64_t invalid : {std::int64_t{-1}, std::int64_t{4}, std::numeric_limits<std::int64_t>::max(),
                               std::numeric_limits<std::int64_t>::min()}) {
    const std::vector<std::int64_t> ids{0, invalid};
    DeviceBuffer picked = upload(ids), out = upload(poison);
    auto invocation = gather->create_invocation(scratch.data(), scratch.size());
    REQUIRE(invocation.has_value());
    auto completion = invocation->submit(fixture().queue, *ConstTensorView::create(source, input),
                                         *ConstTensorView::create(indices, picked), *TensorView::create(result, out));
    REQUIRE(completion.has_value());
    EXPECT(completion->wait().IsOutOfRange());
    EXPECT(download<std::uint64_t>(out, 6) == poison);
    std::vector<std::uint64_t> untouched = poison;
    EXPECT(hyle_oracle_gather(8, data.data(), dims, strides, 2, 0, ids.data(), 1, index_dims, index_strides, 1, 1,
                              untouched.data()) == 1);
    EXPECT(untouched == poison);
  }
  const std::vector<std::int64_t> ids{3, 1};
  DeviceBuffer picked = upload(ids), out = upload(poison);
  auto invocation = gather->create_invocation(scratch.data(), scratch.size());
  REQUIRE(invocation.has_value());
  auto completion = invocation->submit(fixture().queue, *ConstTensorView::create(source, input),
                                       *ConstTensorView::create(indices, picked), *TensorView::create(result, out));
  REQUIRE(completion.has_value());
  EXPECT(completion->wait().ok());
  std::vector<std::uint64_t> want(6);
  EXPECT(hyle_oracle_gather(8, data.data(), dims, strides, 2, 0, ids.data(), 1, index_dims, index_strides, 1, 1, want.data()) == 0);
  EXPECT(want == (std::vector<std::uint64_t>{10, 11, 12, 4, 5, 6}));
  EXPECT(download<std::uint64_t>(out, 6) == want);
}

DEVICE_TEST(CategoricalDrawsTheOraclesIndexAndFailsOnInvalidRows) {
  // tests/compute_models/sampling_fixture.h:262-283: three rows of seven equal weights, then +Inf, NaN
  // and an all -Inf row fail with InvalidArgument, and the same key / draw succeeds again unchanged
  const TensorDesc logits = dense(DataType::kFloat32, {3, 7}), counters = dense(DataType::kUInt32, {3, 4});
  std::vector<std::uint32_t> identities;
  for (std::uint32_t row = 0; row < 3; ++row) {
    const std::uint32_t words[4] = {row * 0x9E3779B9U, 0xFEDCBA98U ^ (row * 17), 73 + row, 0};
    identities.insert(identities.end(), words, words + 4);
  }
  auto draw = prepare(fixture().context, Categorical{true}, logits, counters);
  REQUIRE(draw.has_value());
  EXPECT(draw->output_description(1).value() == dense(DataType::kFloat32, {3}));
  DeviceBuffer scratch = DeviceBuffer::create(draw->workspace_requirement().size).value();
  DeviceBuffer keys = upload(identities);
  auto run = [&](const std::vector<float> &values, std::vector<std::int32_t> *picked, std::vector<float> *scores) {
    DeviceBuffer input = upload(values), ids = upload(std::vector<std::int32_t>(3, -7)), logp = upload(std::vector<float>(3, 0.0F));
    auto invocation = draw->create_invocation(scratch.data(), scratch.size());
    auto completion = invocation->submit(fixture().queue, {*ConstTensorView::create(logits, input), *ConstTensorView::create(counters, keys)},
                                         {*TensorView::create(dense(DataType::kInt32, {3}), ids),
                                          *TensorView::create(dense(DataType::kFloat32, {3}), logp)});
    if (!completion.has_value()) return completion.error();
    Status status = completion->wait();
    *picked = download<std::int32_t>(ids, 3);
    *scores = download<float>(logp, 3);
    return status;
  };
  const std::vector<float> valid(21, 0.25F);
  std::vector<std::int32_t> before, after, want(3);
  std::vector<float> before_scores, after_scores, want_scores(3);
  EXPECT(run(valid, &before, &before_scores).ok());
  EXPECT(hyle_oracle_categorical(HYLE_ORACLE_F32, valid.data(), identities.data(), 3, 7, want.data(), want_scores.data()) == 0);
  EXPECT(before == want);
  for (int row = 0; row < 3; ++row) EXPECT(std::fabs(before_scores[row] - want_scores[row]) <= 2e-5F);
  for (int kind = 0; kind < 3; ++kind) {
    std::vector<float> bad = valid;
    if (kind == 0) bad[9] = std::numeric_limits<float>::infinity();
    if (kind == 1) bad[9] = std::numeric_limits<float>::quiet_NaN();
    if (kind == 2) std::fill(bad.begin() + 7, bad.begin() + 14, -std::numeric_limits<float>::infinity());
    EXPECT(run(bad, &after, &after_scores).IsInvalidArgument());
    EXPECT(hyle_oracle_categorical(HYLE_ORACLE_F32, bad.data(), identities.data(), 3, 7, want.data(), want_scores.data()) == 1);
    EXPECT(run(valid, &after, &after_scores).ok());
    EXPECT(after == before && after_scores == before_scores);
  }
}

DEVICE_TEST(RopeMatchesTheReferenceTestsKnownAnswers) {
  // tests/compute_provider_ggml/cpu_provider_test.cc:1609-1648: f32 [1, 2, 1, 8], positions {0, 2},
  // frequencies {0.5, 0.25}, rotary 4, half-split; in place
  const TensorDesc data = dense(DataType::kFloat32, {1, 2, 1, 8});
  std::vector<float> values(16);
  for (int i = 0; i < 16; ++i) values[i] = static_cast<float>(i + 1);
  auto rope = prepare(fixture().context, RoPE{4, 1, RopeLayout::kHalfSplit}, data, dense(DataType::kInt32, {2}),
                      dense(DataType::kFloat32, {2}));
  REQUIRE(rope.has_value());
  EXPECT(rope->alias_support(0, 0)->supported);
  DeviceBuffer x = upload(values), positions = upload(std::vector<std::int32_t>{0, 2}), frequencies = upload(std::vector<float>{0.5F, 0.25F});
  auto invocation = rope->create_invocation();
  REQUIRE(invocation.has_value());
  auto completion = invocation->submit(fixture().queue, *ConstTensorView::create(data, x),
                                       *ConstTensorView::create(dense(DataType::kInt32, {2}), positions),
                                       *ConstTensorView::create(dense(DataType::kFloat32, {2}), frequencies), *TensorView::create(data, x));
  REQUIRE(completion.has_value());
  EXPECT(completion->wait().ok());
  const std::vector<float> got = download<float>(x, 16);
  std::vector<double> want(16);
  for (int i = 0; i < 16; ++i) want[i] = i + 1;
  want[8] = 9.0 * std::cos(1.0) - 11.0 * std::sin(1.0);
  want[9] = 10.0 * std::cos(0.5) - 12.0 * std::sin(0.5);
  want[10] = 9.0 * std::sin(1.0) + 11.0 * std::cos(1.0);
  want[11] = 10.0 * std::sin(0.5) + 12.0 * std::cos(0.5);
  for (int i = 0; i < 16; ++i) EXPECT(std::fabs(got[i] - want[i]) <= 1e-5);
  std::vector<float> oracle(16);
  const std::int64_t dims[4] = {1, 2, 1, 8};
  const std::int32_t steps[2] = {0, 2};
  const float rates[2] = {0.5F, 0.25F};
  hyle_oracle_rope(HYLE_ORACLE_F32, values.data(), dims, 4, 1, steps, 0, 0, rates, 0, 4, 1, oracle.data());
  for (int i = 0; i < 16; ++i) EXPECT(std::fabs(got[i] - oracle[i]) <= 4e-6F * 24.0F);
}

DEVICE_TEST(RejectedSubmissionsEnqueueNothing) {
  const TensorDesc d = dense(DataType::kFloat32, {8, 64}), row = dense(DataType::kFloat32, {64});
  auto prepared = prepare(fixture().context, Binary{BinaryKind::kMultiply}, d, row);
  REQUIRE(prepared.has_value());
  std::vector<float> ones(512, 1.0F);
  DeviceBuffer a = upload(ones), b = upload(ones), out = DeviceBuffer::create(512 * 4).value();
  auto invocation = prepared->create_invocation().value();
  // One binding short.
  auto short_bound = invocation.submit(fixture().queue, {*ConstTensorView::create(d, a)}, {*TensorView::create(d, out)});
  EXPECT(!short_bound.has_value() && short_bound.error().IsInvalidArgument());
  // The output may share storage with the left input only (its descriptor equals the output's);
  // writing over the broadcast right operand is refused.
  EXPECT(prepared->alias_support(0, 0)->supported && !prepared->alias_support(0, 1)->supported);
  auto aliased = invocation.submit(fixture().queue, *ConstTensorView::create(d, a), *ConstTensorView::create(row, b),
                                   *TensorView::create(d, b));
  EXPECT(!aliased.has_value() && aliased.error().IsInvalidArgument());
  // Storage too small for the description never reaches the provider.
  EXPECT(TensorView::create(d, out.data(), 100).error().IsInvalidArgument());
  // The invocation stays usable after rejections.
  auto completion = invocation.submit(fixture().queue, *ConstTensorView::create(d, a), *ConstTensorView::create(row, b),
                                      *TensorView::create(d, out));
  REQUIRE(completion.has_value());
  EXPECT(completion->wait().ok());
  EXPECT(download<float>(out, 512) == ones);
}

}  // namespace

int main(int argc, char **argv) {
  const bool device = argc > 1 && std::string(argv[1]) == "--device";
  if (argc != 2 || (!device && std::string(argv[1]) != "--host")) {
    std::printf("usage: %s --host | --device\n", argv[0]);
    return 2;
  }
  int ran = 0;
  for (const Case &c : cases()) {
    if (c.device != device) continue;
    std::printf("[ RUN ] %s\n", c.name);
    std::fflush(stdout);
    const int before = failures;
    c.body();
    std::printf("[ %s ] %s\n", failures == before ? " OK " : "FAIL", c.name);
    std::fflush(stdout);
    ++ran;
  }
  std::printf("%d tests, %d failed expectations\n", ran, failures);
  return failures == 0 ? 0 : 1;
}
