// C++ programs written against include/plaidml/* exactly as a user of the reference would write them,
// linked to libplaidml.so and run on the hip device.  Cases and expected values follow the
// reference's own tests (plaidml/edsl/tests/edsl_test.cc: Dot :48-54 / :1203-1252, Max :576-590,
// EltwiseAdd :1181-1201, FunkySum :2709-2719, UseDefault :1148-1164, ArgMax :2126-2137 pattern,
// DotF16_AccF32 pattern :509-545 with int8 -> int32; plaidml/edsl/examples/gemm.cc:66-77).
// Prints "ok <case>" per passing case; exits 1 on the first failure.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <string>
#include <vector>

#include "plaidml/edsl/edsl.h"
#include "plaidml/exec/exec.h"
#include "plaidml/op/op.h"

using namespace plaidml;        // NOLINT
using namespace plaidml::edsl;  // NOLINT

namespace {

template <typename T>
Buffer makeBuffer(DType dt, const std::vector<int64_t>& dims, const std::vector<T>& data) {
  Buffer b(TensorShape(dt, dims));
  b.copy_from(data.data());
  return b;
}

template <typename T>
std::vector<T> readBuffer(Buffer& b) {
  std::vector<T> out(b.size() / sizeof(T));
  b.copy_into(out.data());
  return out;
}

[[noreturn]] void fail(const std::string& name, const std::string& what) {
  std::fprintf(stderr, "FAILED %s: %s\n", name.c_str(), what.c_str());
  std::exit(1);
}

template <typename T>
void expectEq(const std::string& name, const std::vector<T>& got, const std::vector<T>& want) {
  if (got.size() != want.size()) fail(name, "size mismatch");
  for (size_t i = 0; i < got.size(); ++i)
    if (got[i] != want[i]) fail(name, "element " + std::to_string(i) + ": got " + std::to_string(got[i]) + " want " + std::to_string(want[i]));
  std::printf("ok %s\n", name.c_str());
}

void expectClose(const std::string& name, const std::vector<float>& got, const std::vector<float>& want, float rtol, float atol) {
  if (got.size() != want.size()) fail(name, "size mismatch");
  for (size_t i = 0; i < got.size(); ++i)
    if (std::fabs(got[i] - want[i]) > atol + rtol * std::fabs(want[i]))
      fail(name, "element " + std::to_string(i) + ": got " + std::to_string(got[i]) + " want " + std::to_string(want[i]));
  std::printf("ok %s\n", name.c_str());
}

std::vector<Buffer> run(const Program& program_in, std::vector<Buffer> inputs) {
  Program program = program_in;
  program.compile();
  exec::Executable exe(program);
  std::vector<Buffer> outputs;
  for (const TensorShape& shape : program.outputs()) outputs.emplace_back(shape);
  exe.run(inputs, outputs);
  return outputs;
}

Tensor Dot(const Tensor& A, const Tensor& B) {
  TensorDim I, J, K;
  TensorIndex i, j, k;
  A.bind_dims(I, K);
  B.bind_dims(K, J);
  return Contraction().outShape(I, J).outAccess(i, j).sum(A(i, k) * B(k, j));
}

void caseDot() {
  const int64_t M = 8, N = 32, K = 16;
  auto A = Placeholder(DType::FLOAT32, {M, K});
  auto B = Placeholder(DType::FLOAT32, {K, N});
  auto program = buildProgram("dot", {A, B}, {Dot(A, B)});
  std::default_random_engine rng(2);
  std::normal_distribution<float> dist(0.0, 1.0);
  std::vector<float> a(M * K), b(K * N), want(M * N, 0.f);
  for (auto& x : a) x = dist(rng);
  for (auto& x : b) x = dist(rng);
  for (int64_t i = 0; i < M; ++i)
    for (int64_t j = 0; j < N; ++j)
      for (int64_t k = 0; k < K; ++k) want[i * N + j] += a[i * K + k] * b[k * N + j];
  auto out = run(program, {makeBuffer(DType::FLOAT32, {M, K}, a), makeBuffer(DType::FLOAT32, {K, N}, b)});
  expectClose("dot_f32", readBuffer<float>(out[0]), want, 1e-3f, 1e-4f);
}

void caseMax() {
  auto I = Placeholder(DType::FLOAT32, {3, 3});
  TensorDim M, N;
  TensorIndex m, n;
  I.bind_dims(M, N);
  Tensor O = Contraction().outShape(M).outAccess(m).max(I(m, n));
  auto program = buildProgram("max", {I}, {O});
  std::vector<float> in = {-5.0f, -6.0f, -7.0f, 4.0f, 5.0f, 6.0f, 7.0f, 8.0f, 9.0f};
  auto out = run(program, {makeBuffer(DType::FLOAT32, {3, 3}, in)});
  expectEq<float>("max_rows", readBuffer<float>(out[0]), {-5.0f, 6.0f, 9.0f});
}

void caseEltwiseAdd() {
  auto A = Placeholder(DType::FLOAT32, {10, 20});
  auto B = Placeholder(DType::FLOAT32, {10, 20});
  auto program = buildProgram("eltwise_add", {A, B}, {A + B});
  std::vector<float> a(200), b(200), want(200);
  for (int i = 0; i < 200; ++i) {
    a[i] = 0.25f * i;
    b[i] = 100.f - i;
    want[i] = a[i] + b[i];
  }
  auto out = run(program, {makeBuffer(DType::FLOAT32, {10, 20}, a), makeBuffer(DType::FLOAT32, {10, 20}, b)});
  expectEq<float>("eltwise_add", readBuffer<float>(out[0]), want);
}

void caseFunkySum() {
  // O[i] += I[(i - j + 1) / 2] * K[j] on I = K = [1, 2, 3], five outputs  ->  [2, 5, 4, 9, 6]
  auto I = Placeholder(DType::FLOAT32, {3});
  auto Kt = Placeholder(DType::FLOAT32, {3});
  TensorIndex i, j;
  Tensor O = Contraction().outShape(5).outAccess(i).sum(I((i - j + 1) / 2) * Kt(j));
  auto program = buildProgram("funky_sum", {I, Kt}, {O});
  auto out = run(program, {makeBuffer<float>(DType::FLOAT32, {3}, {1, 2, 3}), makeBuffer<float>(DType::FLOAT32, {3}, {1, 2, 3})});
  expectEq<float>("funky_sum", readBuffer<float>(out[0]), {2, 5, 4, 9, 6});
}

void caseUseDefault() {
  // O[b, 3, i1, i2] = I[b, i1, i2] over a default tensor P
  auto P = Placeholder(DType::FLOAT32, {1, 7, 10, 10});
  auto I = Placeholder(DType::FLOAT32, {1, 10, 10});
  TensorDim B, N1, N2;
  TensorIndex b, i1, i2;
  I.bind_dims(B, N1, N2);
  Tensor O = Contraction().outShape(B, 7, N1, N2).outAccess(b, 3, i1, i2).assign(I(b, i1, i2)).init(P);
  auto program = buildProgram("use_default", {I, P}, {O});
  std::vector<float> p(700), in(100), want(700);
  for (int k = 0; k < 700; ++k) want[k] = p[k] = 0.5f * k;
  for (int k = 0; k < 100; ++k) want[300 + k] = in[k] = -1.f - k;
  auto out = run(program, {makeBuffer(DType::FLOAT32, {1, 10, 10}, in), makeBuffer(DType::FLOAT32, {1, 7, 10, 10}, p)});
  expectEq<float>("use_default", readBuffer<float>(out[0]), want);
}

void caseInt8Gemm() {
  // int8 x int8 accumulated in int32: the cast comes before the contraction
  const int64_t M = 64, N = 48, K = 32;
  auto A = Placeholder(DType::INT8, {M, K});
  auto B = Placeholder(DType::INT8, {K, N});
  auto program = buildProgram("gemm_i8", {A, B}, {Dot(cast(A, DType::INT32), cast(B, DType::INT32))});
  std::default_random_engine rng(4);
  std::uniform_int_distribution<int> dist(-127, 127);
  std::vector<int8_t> a(M * K), b(K * N);
  std::vector<int32_t> want(M * N, 0);
  for (auto& x : a) x = static_cast<int8_t>(dist(rng));
  for (auto& x : b) x = static_cast<int8_t>(dist(rng));
  for (int64_t i = 0; i < M; ++i)
    for (int64_t j = 0; j < N; ++j)
      for (int64_t k = 0; k < K; ++k) want[i * N + j] += static_cast<int32_t>(a[i * K + k]) * b[k * N + j];
  auto out = run(program, {makeBuffer(DType::INT8, {M, K}, a), makeBuffer(DType::INT8, {K, N}, b)});
  expectEq<int32_t>("gemm_i8_i32", readBuffer<int32_t>(out[0]), want);
}

void caseConvRelu() {
  // op::relu(op::convolution(I, F) + B): NXC / XCK / SAME_UPPER / stride 1 defaults
  const int64_t N = 2, H = 9, W = 11, CI = 32, CO = 48;
  auto I = Placeholder(DType::FLOAT32, {N, H, W, CI});
  auto F = Placeholder(DType::FLOAT32, {3, 3, CI, CO});
  auto Bv = Placeholder(DType::FLOAT32, {CO});
  Tensor O = op::relu(op::convolution(I, F) + Bv);
  auto program = buildProgram("conv_relu", {I, F, Bv}, {O});
  std::default_random_engine rng(7);
  std::normal_distribution<float> dist(0.0, 1.0);
  std::vector<float> in(N * H * W * CI), f(9 * CI * CO), bias(CO), want(N * H * W * CO);
  for (auto& x : in) x = dist(rng);
  for (auto& x : f) x = 0.1f * dist(rng);
  for (auto& x : bias) x = dist(rng);
  for (int64_t n = 0; n < N; ++n)
    for (int64_t y = 0; y < H; ++y)
      for (int64_t x = 0; x < W; ++x)
        for (int64_t co = 0; co < CO; ++co) {
          double acc = bias[co];
          for (int64_t ky = 0; ky < 3; ++ky)
            for (int64_t kx = 0; kx < 3; ++kx) {
              const int64_t iy = y + ky - 1, ix = x + kx - 1;
              if (iy < 0 || iy >= H || ix < 0 || ix >= W) continue;
              for (int64_t ci = 0; ci < CI; ++ci)
                acc += static_cast<double>(in[((n * H + iy) * W + ix) * CI + ci]) * f[((ky * 3 + kx) * CI + ci) * CO + co];
            }
          want[((n * H + y) * W + x) * CO + co] = acc < 0 ? 0.f : static_cast<float>(acc);
        }
  auto out = run(program, {makeBuffer(DType::FLOAT32, {N, H, W, CI}, in), makeBuffer(DType::FLOAT32, {3, 3, CI, CO}, f),
                           makeBuffer(DType::FLOAT32, {CO}, bias)});
  expectClose("conv_bias_relu", readBuffer<float>(out[0]), want, 1e-3f, 1e-4f);
}

// op library data movement, written as plaidml/op/op_test.cc writes it (ExplicitPadding :318-333,
// ExplicitPaddingEdge :385-418, CumSumExclusive :297-304, Transpose / Concatenate patterns :174-180,698-702)
void caseOpLibrary() {
  {
    auto I = Placeholder(DType::FLOAT32, {2, 3});
    Tensor O = op::explicit_padding(I, {2, 1}, {2, 1}).mode(op::PadMode::CONSTANT).padval(Constant(-1.0));
    auto program = buildProgram("explicit_padding", {I}, {O});
    auto out = run(program, {makeBuffer<float>(DType::FLOAT32, {2, 3}, {1, 2, 3, 4, 5, 6})});
    expectEq<float>("explicit_padding", readBuffer<float>(out[0]),
                    {-1, -1, -1, -1, -1, -1, -1, -1, -1, -1, -1, 1, 2, 3, -1, -1, 4, 5, 6, -1, -1, -1, -1, -1, -1, -1, -1, -1, -1, -1});
  }
  {
    auto I = Placeholder(DType::FLOAT32, {1, 2, 3});
    Tensor O = op::explicit_padding(I, {1, 2, 1}, {2, 1, 3}).mode(op::PadMode::EDGE);
    auto program = buildProgram("explicit_padding_edge", {I}, {O});
    auto out = run(program, {makeBuffer<float>(DType::FLOAT32, {1, 2, 3}, {1, 2, 3, 4, 5, 6})});
    std::vector<float> want;
    for (int n = 0; n < 4; ++n)
      for (int r = 0; r < 5; ++r) {
        const std::vector<float> row = r < 3 ? std::vector<float>{1, 1, 2, 3, 3, 3, 3} : std::vector<float>{4, 4, 5, 6, 6, 6, 6};
        want.insert(want.end(), row.begin(), row.end());
      }
    expectEq<float>("explicit_padding_edge", readBuffer<float>(out[0]), want);
  }
  {
    auto I = Placeholder(DType::FLOAT32, {4});
    auto program = buildProgram("cumsum", {I}, {op::cumsum(I, 0, true)});
    auto out = run(program, {makeBuffer<float>(DType::FLOAT32, {4}, {2, 4, 6, 8})});
    expectEq<float>("cumsum_exclusive", readBuffer<float>(out[0]), {0, 2, 6, 12});
  }
  {
    auto A = Placeholder(DType::FLOAT32, {2, 3});
    auto B = Placeholder(DType::FLOAT32, {2, 2});
    Tensor O = op::transpose(op::concatenate({A, B}, 1), edsl::make_tuple(std::vector<int64_t>{1, 0}));
    auto program = buildProgram("concat_transpose", {A, B}, {O});
    auto out = run(program, {makeBuffer<float>(DType::FLOAT32, {2, 3}, {1, 2, 3, 4, 5, 6}),
                             makeBuffer<float>(DType::FLOAT32, {2, 2}, {7, 8, 9, 10})});
    expectEq<float>("concat_transpose", readBuffer<float>(out[0]), {1, 4, 2, 5, 3, 6, 7, 9, 8, 10});
  }
}

// Operators and libm intrinsics of the header, with the reference's own answers
// (plaidml/edsl/tests/edsl_test.cc: BitRightScalar :273-287, BitNot :289-302, EltwiseMod :606-629,
// LogicalAnd_mixed :1223-1241, LogicalNot_float :1315-1328, Pow :1796-1817, Tan :1857-1873).
void caseIntrinsics() {
  {
    auto A = Placeholder(DType::UINT64, {3, 3});
    std::vector<uint64_t> a, want;
    for (uint64_t k = 1; k <= 9; ++k) {
      a.push_back(k << (9 + k));
      want.push_back(k << k);
    }
    auto out = run(buildProgram("bit_right_scalar", {A}, {A >> 9}), {makeBuffer<uint64_t>(DType::UINT64, {3, 3}, a)});
    expectEq<uint64_t>("bit_right_scalar", readBuffer<uint64_t>(out[0]), want);
  }
  {
    auto A = Placeholder(DType::UINT8, {3, 3});
    auto out = run(buildProgram("bit_not", {A}, {~A}),
                   {makeBuffer<uint8_t>(DType::UINT8, {3, 3}, {0x00, 0x01, 0x02, 0x10, 0x11, 0x22, 0xF0, 0x0F, 0xFF})});
    expectEq<uint8_t>("bit_not", readBuffer<uint8_t>(out[0]), {0xFF, 0xFE, 0xFD, 0xEF, 0xEE, 0xDD, 0x0F, 0xF0, 0x00});
  }
  {
    auto A = Placeholder(DType::INT32, {3, 3});
    auto B = Placeholder(DType::INT32, {3, 3});
    auto out = run(buildProgram("mod", {A, B}, {A % B}), {makeBuffer<int32_t>(DType::INT32, {3, 3}, {2, 4, 8, 16, 32, 64, 128, 256, 512}),
                                                          makeBuffer<int32_t>(DType::INT32, {3, 3}, {1, 2, 3, 4, 5, 6, 7, 8, 9})});
    expectEq<int32_t>("mod", readBuffer<int32_t>(out[0]), {2 % 1, 4 % 2, 8 % 3, 16 % 4, 32 % 5, 64 % 6, 128 % 7, 256 % 8, 512 % 9});
  }
  {
    auto A = Placeholder(DType::UINT64, {3, 3});
    auto B = Placeholder(DType::FLOAT32, {3, 3});
    auto out = run(buildProgram("logical_and", {A, B}, {A && B, !B}),
                   {makeBuffer<uint64_t>(DType::UINT64, {3, 3}, {1, 2, 3, 4, 0, 6, 7, 0, 9}),
                    makeBuffer<float>(DType::FLOAT32, {3, 3}, {10, 11, 12, 13, 0, 15, 16, 17, 18})});
    expectEq<int8_t>("logical_and_mixed", readBuffer<int8_t>(out[0]), {1, 1, 1, 1, 0, 1, 1, 0, 1});
    expectEq<int8_t>("logical_not_float", readBuffer<int8_t>(out[1]), {0, 0, 0, 0, 1, 0, 0, 0, 0});
  }
  {
    auto A = Placeholder(DType::FLOAT32, {3, 3});
    auto B = Placeholder(DType::FLOAT32, {3, 3});
    auto out = run(buildProgram("pow_tan", {A, B}, {pow(A, B), tan(B * 0.4)}),
                   {makeBuffer<float>(DType::FLOAT32, {3, 3}, {0.5, 1.5, 2.5, 0.5, 1.5, 2.5, 0.5, 1.5, 2.5}),
                    makeBuffer<float>(DType::FLOAT32, {3, 3}, {0.5, 0.5, 0.5, 1.5, 1.5, 1.5, 2.5, 2.5, 2.5})});
    expectClose("pow", readBuffer<float>(out[0]), {0.707107, 1.22474, 1.58114, 0.353553, 1.83712, 3.95285, 0.176777, 2.75568, 9.88212},
                2e-5f, 0.f);
    expectClose("tan", readBuffer<float>(out[1]), {0.20271, 0.20271, 0.20271, 0.684137, 0.684137, 0.684137, 1.55741, 1.55741, 1.55741},
                2e-4f, 0.f);
  }
}

// Builder classes of the op header: slice (int and (start, stop, step) entries), broadcast with the reference's
// own case (plaidml/op/op_test.cc:115-127), l2norm, lrn, mvn, reorg_yolo shapes.
void caseOpBuilders() {
  auto A = Placeholder(DType::FLOAT32, {3, 4});
  std::vector<float> a = {0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11};
  {
    Tensor S = op::slice(A).add_dim(1, 3).add_dim(edsl::Value(edsl::None()), edsl::Value(edsl::None()), edsl::Value(-2));
    Tensor R = op::slice(A).add_dim(-1).add_dim(0, 4, 3);
    auto out = run(buildProgram("slice", {A}, {S, R}), {makeBuffer<float>(DType::FLOAT32, {3, 4}, a)});
    expectEq<float>("slice_steps", readBuffer<float>(out[0]), {7, 5, 11, 9});
    expectEq<float>("slice_int", readBuffer<float>(out[1]), {8, 11});
  }
  {
    auto B = Placeholder(DType::FLOAT32, {3, 1});
    auto out = run(buildProgram("broadcast", {B}, {op::broadcast(B, {3, 4}, {0, 1})}), {makeBuffer<float>(DType::FLOAT32, {3, 1}, {0, 1, 2})});
    expectEq<float>("broadcast_numpy2", readBuffer<float>(out[0]), {0, 0, 0, 0, 1, 1, 1, 1, 2, 2, 2, 2});
  }
  {
    Tensor N = op::l2norm(A, {1}).epsilon(1.0f).eps_mode(op::EpsMode::MAX);
    Tensor L = op::lrn(A, {3}).alpha(0.0).beta(2.0).epsilon(2.0);  // x / (0 + 2)^2
    Tensor M = op::mvn(A).axes({1}).normalize_variance(false);
    auto out = run(buildProgram("norms", {A}, {N, L, M}), {makeBuffer<float>(DType::FLOAT32, {3, 4}, a)});
    expectClose("l2norm", readBuffer<float>(out[0]), {std::sqrt(14.f), std::sqrt(126.f), std::sqrt(366.f)}, 1e-5f, 0.f);
    std::vector<float> quarter;
    for (float v : a) quarter.push_back(v / 4);
    expectClose("lrn", readBuffer<float>(out[1]), quarter, 1e-6f, 0.f);
    expectClose("mvn", readBuffer<float>(out[2]), {-1.5, -.5, .5, 1.5, -1.5, -.5, .5, 1.5, -1.5, -.5, .5, 1.5}, 1e-6f, 1e-6f);
  }
  {
    // three boxes of one class: the second overlaps the first (IoU 0.9 / 1.1) and loses, the third stands alone
    auto Bx = Placeholder(DType::FLOAT32, {1, 3, 4});
    auto Sc = Placeholder(DType::FLOAT32, {1, 1, 3});
    auto It = Placeholder(DType::FLOAT32, {1});
    auto St = Placeholder(DType::FLOAT32, {1});
    auto R = op::nms(Bx, Sc, It, St, 3).build();
    auto out = run(buildProgram("nms", {Bx, Sc, It, St}, R),
                   {makeBuffer<float>(DType::FLOAT32, {1, 3, 4}, {0, 0, 1, 1, 0, 0.1f, 1, 1.1f, 2, 2, 3, 3}),
                    makeBuffer<float>(DType::FLOAT32, {1, 1, 3}, {0.9f, 0.8f, 0.7f}), makeBuffer<float>(DType::FLOAT32, {1}, {0.5f}),
                    makeBuffer<float>(DType::FLOAT32, {1}, {0.0f})});
    expectEq<int32_t>("nms_boxes", readBuffer<int32_t>(out[0]), {0, 0, 0, 0, 0, 2, -1, -1, -1});
    expectEq<float>("nms_scores", readBuffer<float>(out[1]), {0, 0, 0.9f, 0, 0, 0.7f, -1, -1, -1});
    expectEq<int32_t>("nms_valid", readBuffer<int32_t>(out[2]), {2});
  }
  {
    auto I = Placeholder(DType::INT64, {1, 4, 6, 6});
    Tensor O = op::reorg_yolo(I, 2, /*decrease=*/false);
    auto dims = O.compute_shape().sizes();
    if (dims != std::vector<int64_t>{1, 16, 3, 3}) fail("reorg_yolo_shape", "unexpected result shape");
    std::printf("ok reorg_yolo_shape\n");
  }
}

// argsort / gather / scatter and the operations built on them, with the reference's answers
// (plaidml/edsl/tests/edsl_test.cc: Gather :1490-1508, InterpolatedGatherLinear :1523-1533, ScatterDup1D :1917-1930,
// ScatterElt :2080-2107, ArgSort1dDup :2462-2492; plaidml/op/op_test.cc: Sort :638-658).
void caseSpecialOps() {
  {
    auto A = Placeholder(DType::FLOAT32, {3, 2});
    auto B = Placeholder(DType::INT32, {4});
    Tensor O = gather(A, B).axis(1);
    auto out = run(buildProgram("gather", {A, B}, {O}),
                   {makeBuffer<float>(DType::FLOAT32, {3, 2}, {-5, -6, -7, 4, 5, 6}), makeBuffer<int32_t>(DType::INT32, {4}, {0, 1, 1, 0})});
    expectEq<float>("gather", readBuffer<float>(out[0]), {-5, -6, -6, -5, -7, 4, 4, -7, 5, 6, 6, 5});
  }
  {
    auto A = Placeholder(DType::FLOAT32, {1, 6});
    auto B = Placeholder(DType::FLOAT32, {12});
    Tensor O = gather(A, B).axis(-1).interpolationMode(InterpolationMode::LINEAR).outOfBoundsMode(OutOfBoundsMode::RETURN_ZERO);
    auto out = run(buildProgram("gather_linear", {A, B}, {O}),
                   {makeBuffer<float>(DType::FLOAT32, {1, 6}, {0, 1, 8, 5, 5, 2}),
                    makeBuffer<float>(DType::FLOAT32, {12}, {-0.25, 0.25, 0.75, 1.25, 1.75, 2.25, 2.75, 3.25, 3.75, 4.25, 4.75, 5.25})});
    expectEq<float>("gather_linear_return_zero", readBuffer<float>(out[0]), {0, 0.25, 0.75, 2.75, 6.25, 7.25, 5.75, 5, 5, 4.25, 2.75, 0});
  }
  {
    auto D = Placeholder(DType::FLOAT32, {8});
    auto I = Placeholder(DType::INT32, {4});
    auto U = Placeholder(DType::FLOAT32, {4});
    Tensor O = scatter(D, I, U);
    auto out = run(buildProgram("scatter", {D, I, U}, {O}),
                   {makeBuffer<float>(DType::FLOAT32, {8}, {0, 0, 0, 0, 0, 0, 0, 0}), makeBuffer<int32_t>(DType::INT32, {4}, {4, 3, 3, 7}),
                    makeBuffer<float>(DType::FLOAT32, {4}, {9, 10, 11, 12})});
    expectEq<float>("scatter_dup", readBuffer<float>(out[0]), {0, 0, 0, 21, 9, 0, 0, 12});
  }
  {
    auto D = Placeholder(DType::FLOAT32, {4, 4});
    auto I = Placeholder(DType::INT32, {2, 2});
    auto U = Placeholder(DType::FLOAT32, {2, 2});
    Tensor O = scatter(D, I, U).axis(1).mode(ScatterMode::UPDATE_ELT);
    auto out = run(buildProgram("scatter_elt", {D, I, U}, {O}),
                   {makeBuffer<float>(DType::FLOAT32, {4, 4}, std::vector<float>(16, 1.f)), makeBuffer<int32_t>(DType::INT32, {2, 2}, {2, 0, 3, 1}),
                    makeBuffer<float>(DType::FLOAT32, {2, 2}, {9, 9, 9, 9})});
    expectEq<float>("scatter_elt", readBuffer<float>(out[0]), {9, 1, 9, 1, 1, 9, 1, 9, 1, 1, 1, 1, 1, 1, 1, 1});
  }
  {
    std::vector<float> x = {81.69, 81.69, 27.74, 43.69, 55.79, 56.79, 57.52, 7.11, 39.48, 5.9,
                            14.81, 66.23, 20.25, 66.05, 64.5,  71.07, 67.6,  54.42, 87.59, 80.02};
    auto I = Placeholder(DType::FLOAT32, {20});
    auto out = run(buildProgram("argsort", {I}, {argsort(I, 0)}), {makeBuffer<float>(DType::FLOAT32, {20}, x)});
    expectEq<int32_t>("argsort_dup", readBuffer<int32_t>(out[0]), {9, 7, 10, 12, 2, 8, 3, 17, 4, 5, 6, 14, 13, 11, 16, 15, 19, 0, 1, 18});
    auto A = Placeholder(DType::FLOAT32, {5, 4});
    auto top = op::topk(A, 2).axis(1).build();
    auto res = run(buildProgram("sort_topk", {A}, {op::sort(A, 1, SortDirection::ASC), top[0], top[1]}),
                   {makeBuffer<float>(DType::FLOAT32, {5, 4}, {81.69, 95.74, 27.74, 43.69, 55.79, 56.79, 57.52, 5.9, 39.48, 7.11,
                                                                14.81, 66.23, 20.25, 66.05, 64.5,  71.07, 67.6,  54.42, 87.59, 80.02})});
    expectEq<float>("sort", readBuffer<float>(res[0]), {27.74, 43.69, 81.69, 95.74, 5.9,   55.79, 56.79, 57.52, 7.11,  14.81,
                                                        39.48, 66.23, 20.25, 64.5,  66.05, 71.07, 54.42, 67.6,  80.02, 87.59});
    expectEq<float>("topk_values", readBuffer<float>(res[1]), {95.74, 81.69, 57.52, 56.79, 66.23, 39.48, 71.07, 66.05, 87.59, 80.02});
    expectEq<int32_t>("topk_positions", readBuffer<int32_t>(res[2]), {1, 0, 2, 1, 3, 0, 3, 1, 2, 3});
  }
}

// CppEdsl.Lens, plaidml/edsl/tests/edsl_test.cc:2122-2162: a transposition written once for "MN" and read through a
// lens gives the same answer whichever of the two orders names the tensor's own layout
Tensor TransposeThroughLens(Tensor I, const std::string& layout) {
  TensorLens lens(layout, "MN");
  I = I.use(lens);
  TensorDim M, N;
  TensorIndex i, j;
  I.bind_dims(M, N);
  return Contraction(lens).outShape(N, M).outAccess(j, i).assign(I(i, j));
}

void caseLens() {
  for (const char* layout : {"MN", "NM"}) {
    auto I = Placeholder(DType::FLOAT32, {2, 3});
    auto out = run(buildProgram("transpose", {I}, {TransposeThroughLens(I, layout)}), {makeBuffer<float>(DType::FLOAT32, {2, 3}, {1, 2, 3, 4, 5, 6})});
    expectEq<float>(std::string("lens_transpose_") + layout, readBuffer<float>(out[0]), {1, 4, 2, 5, 3, 6});
  }
}

void caseErrors() {
  auto A = Placeholder(DType::FLOAT32, {4, 4});
  auto program = buildProgram("ident", {A}, {A + 1.0});
  program.compile();
  exec::Executable exe(program);
  Buffer out(TensorShape(DType::FLOAT32, {4, 4}));
  try {
    exe.run({}, {out});
  } catch (const std::exception& e) {
    if (std::string(e.what()).find("Program expects 1 inputs, but 0 were specified") == std::string::npos)
      fail("arity_error", std::string("unexpected text: ") + e.what());
    std::printf("ok arity_error\n");
    return;
  }
  fail("arity_error", "no exception");
}

template <typename F>
void expectThrows(const char* name, F&& fn) {
  try {
    fn();
  } catch (const std::exception&) {
    std::printf("ok %s\n", name);
    return;
  }
  fail(name, "no exception");
}

// The misuse cases of plaidml/edsl/tests/edsl_test.cc:2274-2398 and its layer / trace cases (:2110-2345).
void caseReferenceErrors() {
  expectThrows("bad_data_type", [] { auto A = Placeholder(DType::INVALID, {10, 20}); });
  expectThrows("index_without_dims", [] { plaidml::edsl::index(std::vector<TensorDim>{}, 0); });
  expectThrows("index_unbound_dim", [] {
    TensorDim X0;
    plaidml::edsl::index({X0}, 0);
  });
  {
    TensorDim X0, X1;
    auto I = Placeholder(DType::FLOAT32, {10, 3});
    I.bind_dims(X0, X1);
    Tensor O = plaidml::edsl::index({X0}, 0);
    auto out = run(buildProgram("IndexOp", {}, {O}), {});
    expectEq<int32_t>("index_op", readBuffer<int32_t>(out[0]), {0, 1, 2, 3, 4, 5, 6, 7, 8, 9});
  }
  expectThrows("bind_bad_dims", [] {
    auto X = Placeholder(DType::FLOAT32, {10, 10});
    auto Y = Placeholder(DType::FLOAT32, {12, 10});
    TensorDim I, J, K;
    X.bind_dims({I, K});
    Y.bind_dims({K, J});
  });
  expectThrows("eltwise_mismatch", [] {
    auto X = Placeholder(DType::FLOAT32, {10, 10});
    auto Y = Placeholder(DType::FLOAT32, {12, 10});
    auto O = X + Y;
  });
  expectThrows("op_operators", [] {
    auto X = Placeholder(DType::FLOAT32, {10, 10});
    auto Y = Placeholder(DType::FLOAT32, {12, 12});
    auto O = op::relu(X) + op::relu(Y);
  });
  {
    auto A = Placeholder(DType::FLOAT32, {2, 2});
    expectThrows("layer_exception", [&] { layer("sum", {A}, [&]() -> Tensor { throw std::runtime_error("exception"); }); });
    Tensor B = layer("sum", {A}, [&]() { return A + Constant(makeBuffer<float>(DType::FLOAT32, {2, 2}, {1, 2, 3, 4}), "C"); });
    Tensor O = layer("sum", {B}, [&]() { return trace(B, "msg") + Constant(makeBuffer<float>(DType::FLOAT32, {2, 2}, {1, 2, 3, 4}), "C"); });
    auto out = run(buildProgram("LayerMulti", {A}, {O}), {makeBuffer<float>(DType::FLOAT32, {2, 2}, {10, 20, 30, 40})});
    expectEq<float>("layer_multi", readBuffer<float>(out[0]), {12, 24, 36, 48});
  }
  {
    auto A = Placeholder(DType::FLOAT32, {3, 2});
    TensorVec both = layer("two_output", {A}, {}, [&]() {
      Tensor idxs = argsort(A, 0);
      Tensor vals = gather(A, idxs);
      return TensorVec{vals, idxs};
    });
    auto out = run(buildProgram("LayerMultipleReturnValues", {A}, both), {makeBuffer<float>(DType::FLOAT32, {3, 2}, {3, 9, 1, 8, 2, 7})});
    expectEq<int32_t>("layer_two_outputs_positions", readBuffer<int32_t>(out[1]), {1, 2, 2, 1, 0, 0});
  }
}

}  // namespace

int main() {
  plaidml::init();
  plaidml::edsl::init();
  plaidml::op::init();
  plaidml::exec::init();
  Settings::set("PLAIDML_DEVICE", "hip.0");
  Settings::set("PLAIDML_TARGET", "hip");
  try {
    caseDot();
    caseMax();
    caseEltwiseAdd();
    caseFunkySum();
    caseUseDefault();
    caseInt8Gemm();
    caseConvRelu();
    caseOpLibrary();
    caseIntrinsics();
    caseOpBuilders();
    caseSpecialOps();
    caseLens();
    caseErrors();
    caseReferenceErrors();
  } catch (const std::exception& e) {
    std::fprintf(stderr, "FAILED with exception: %s\n", e.what());
    return 1;
  }
  std::printf("all cases passed\n");
  return 0;
}
