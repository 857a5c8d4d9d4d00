// GPU test of the C++ host layer: tensors, registration, HipAutogradExtension and
// the caller closures, checked against the CPU checker (oracle/flref.c).  The
// cases re-express the reference's own tests for this path:
//   flashlight/fl/test/tensor/TensorExtensionTest.cpp:24-68 (extension reachable),
//   flashlight/fl/test/autograd/AutogradConv2DTest.cpp:21-74,137-162 (shapes),
//   flashlight/fl/test/autograd/AutogradTest.cpp:65-81,333-337 (dtype errors, pool),
//   flashlight/fl/test/autograd/AutogradNormalizationTest.cpp:158-189 (batchnorm),
//   flashlight/fl/test/nn/ModuleTest.cpp:338-353 (batching invariance),
// one training step of the README MNIST convnet (README.md:45-84) through the tape, and
// the nn modules over those functions (flashlight/fl/test/nn/ModuleTest.cpp:670-719 for
// LayerNorm; Sequential, BatchNorm statistics, a ResNet bottleneck with its residual add,
// the 21x1 convolution / batch norm / ReLU stack of the speech configuration).
#include <algorithm>
#include <cmath>
#include <csignal>
#include <execinfo.h>
#include <unistd.h>
#include <cstdio>
#include <cstring>
#include <functional>
#include <map>
#include <random>
#include <string>
#include <unordered_set>
#include <vector>

#include "Functions.h"
#include "Modules.h"
#include "Optimizers.h"
#include "SequentialBuilder.h"
#include "HipAutogradExtension.h"
#include "OpObserver.h"
#include "DynamicBenchmark.h"
#include "flhip.h"
#include "flref.h"

using namespace fl;

static int g_fail = 0;
#define CHECK(cond)                                                          \
  do {                                                                       \
    if (!(cond)) {                                                           \
      std::printf("  FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);        \
      ++g_fail;                                                              \
    }                                                                        \
  } while (0)

static std::vector<float> randn(size_t n, unsigned seed, float scale = 1.f, float shift = 0.f) {
  std::mt19937 gen(seed);
  std::normal_distribution<float> d(0.f, 1.f);
  std::vector<float> v(n);
  for (auto& x : v) x = d(gen) * scale + shift;
  return v;
}
static double relL2(const std::vector<float>& a, const std::vector<float>& b) {
  double num = 0, den = 0;
  if (a.size() != b.size()) return 1e30;
  for (size_t i = 0; i < a.size(); ++i) {
    num += ((double)a[i] - b[i]) * ((double)a[i] - b[i]);
    den += (double)b[i] * b[i];
  }
  return den > 0 ? std::sqrt(num / den) : std::sqrt(num);
}
static double maxAbsDiff(const std::vector<float>& a, const std::vector<float>& b) {
  double m = a.size() == b.size() ? 0 : 1e30;
  for (size_t i = 0; i < a.size() && i < b.size(); ++i) m = std::max(m, std::fabs((double)a[i] - b[i]));
  return m;
}
static float bf16round(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  u &= 0xffff0000u;
  std::memcpy(&f, &u, 4);
  return f;
}
// nearest IEEE half value (ties to even), as a float
static float f16round(float f) {
  if (!std::isfinite(f) || f == 0.f) return f;
  const float a = std::fabs(f);
  if (a >= 65520.f) return std::copysign(INFINITY, f);
  int e;
  std::frexp(a, &e);                                   // a = m * 2^e, m in [0.5, 1)
  const int q = e - 11 < -24 ? -24 : e - 11;           // 11 significant bits; subnormals step by 2^-24
  return std::copysign(std::ldexp(std::nearbyint(std::ldexp(a, -q)), q), f);
}
static float roundTo(dtype dt, float f) { return dt == dtype::bf16 ? bf16round(f) : dt == dtype::f16 ? f16round(f) : f; }
template <typename E>
static bool throws(const std::function<void()>& f) {
  try {
    f();
  } catch (const E&) {
    return true;
  } catch (...) {
    return false;
  }
  return false;
}

static void testRegistration() {
  std::printf("registration\n");
  AutogradExtension& e = getAutogradExtension(TensorBackendType::Hip);
  CHECK(dynamic_cast<HipAutogradExtension*>(&e) != nullptr);
  CHECK(&e == &getAutogradExtension(TensorBackendType::Hip));       // one instance per backend
  CHECK(e.isDataTypeSupported(dtype::f32) && e.isDataTypeSupported(dtype::bf16) && e.isDataTypeSupported(dtype::f16));
  CHECK(!e.isDataTypeSupported(dtype::f64) && !e.isDataTypeSupported(dtype::s32));
  CHECK(e.createBenchmarkOptions() != nullptr && e.createBenchmarkOptions() != e.createBenchmarkOptions());   // one per pass and layer
  // a second registration for the same backend is ignored (TensorExtension.cpp:27-29)
  CHECK(!detail::registerAutogradExtension(TensorBackendType::Hip, [] {
    return std::unique_ptr<AutogradExtension>(new HipAutogradExtension());
  }));
  CHECK(throws<std::invalid_argument>([] { getAutogradExtension(TensorBackendType::Stub); }));
  CHECK(throws<std::runtime_error>([&] {   // an empty input
    Tensor t;
    e.rnn(t, t, t, t, 1, 1, RnnMode::LSTM, false, 0.f, nullptr);
  }));
}

static void testConv(dtype dt, int groups, double tol) {
  std::printf("conv2d %s groups=%d\n", dt == dtype::f32 ? "f32" : dt == dtype::bf16 ? "bf16" : "f16", groups);
  // input [10,9,8,7], weights [4,3,8/groups,6], px=2, py=1
  const int W = 10, H = 9, C = 8, N = 7, KW = 4, KH = 3, K = 6, px = 2, py = 1;
  flref_conv d{N, C, H, W, K, KH, KW, 1, 1, py, px, 1, 1, groups};
  int32_t OH, OW;
  flref_conv_out(&d, &OH, &OW);
  auto x = randn((size_t)N * C * H * W, 1), w = randn((size_t)K * (C / groups) * KH * KW, 2, 0.2f);
  auto b = randn(K, 3), dy = randn((size_t)N * K * OH * OW, 4);
  for (auto* v : {&x, &w, &b, &dy})
    for (auto& f : *v) f = roundTo(dt, f);
  std::vector<float> y(dy.size()), dx(x.size()), dw(w.size()), db(K);
  flref_conv2d_fwd(&d, x.data(), w.data(), b.data(), y.data());
  flref_conv2d_bwd_data(&d, dy.data(), w.data(), dx.data());
  flref_conv2d_bwd_filter(&d, x.data(), dy.data(), dw.data(), db.data());

  Variable in(Tensor::fromVector({W, H, C, N}, x).astype(dt), true);
  Variable wt(Tensor::fromVector({KW, KH, C / groups, K}, w).astype(dt), true);
  Variable bs(Tensor::fromVector({1, 1, K, 1}, b).astype(dt), true);
  Variable out = conv2d(in, wt, bs, 1, 1, px, py, 1, 1, groups);
  CHECK(out.shape() == Shape({OW, OH, K, N}));
  CHECK(out.type() == dt);
  CHECK(relL2(out.tensor().toHostVector(), y) <= tol);
  out.backward(Variable(Tensor::fromVector(out.shape(), dy).astype(dt), false));
  CHECK(relL2(in.grad().tensor().toHostVector(), dx) <= tol);
  CHECK(relL2(wt.grad().tensor().toHostVector(), dw) <= tol);
  CHECK(relL2(bs.grad().tensor().toHostVector(), db) <= tol);
  CHECK(in.grad().type() == dt && wt.grad().type() == dt && bs.grad().shape() == bs.shape());

  // an input without gradient: backward-data is skipped (Functions.cpp:1407)
  Variable in2(in.tensor(), false), wt2(wt.tensor(), true);
  Variable out2 = conv2d(in2, wt2, 1, 1, px, py, 1, 1, groups);
  out2.backward(Variable(Tensor::fromVector(out2.shape(), dy).astype(dt), false));
  CHECK(!in2.isGradAvailable() && wt2.isGradAvailable());
  CHECK(relL2(wt2.grad().tensor().toHostVector(), dw) <= tol);
}

static void testConvErrors() {
  std::printf("conv2d errors\n");
  Variable in(Tensor({8, 8, 4, 1}, dtype::f32), false);
  Variable wbf(Tensor({3, 3, 4, 4}, dtype::bf16), false);
  // mixed types are rejected before the boundary (AutogradTest.cpp:75-81)
  CHECK(throws<std::invalid_argument>([&] { conv2d(in, wbf); }));
  Variable wbad(Tensor({3, 3, 3, 4}, dtype::f32), false);
  CHECK(throws<std::invalid_argument>([&] { conv2d(in, wbad); }));
  Variable wbig(Tensor({9, 9, 4, 4}, dtype::f32), false);
  CHECK(throws<std::invalid_argument>([&] { conv2d(in, wbig); }));
  Variable f64(Tensor({8, 8, 4, 1}, dtype::f64), false), w64(Tensor({3, 3, 4, 4}, dtype::f64), false);
  CHECK(throws<std::runtime_error>([&] { conv2d(f64, w64); }));
}

static void testBatchingInvariance() {
  std::printf("conv2d batching invariance\n");
  // 30 -> 50 channels, 9x7 kernel, stride 2x3, padding 3x2 (ModuleTest.cpp:338-353)
  const int W = 20, H = 17, C = 30, N = 4, K = 50;
  auto x = randn((size_t)N * C * H * W, 5), w = randn((size_t)K * C * 7 * 9, 6, 0.03f);
  Variable wt(Tensor::fromVector({9, 7, C, K}, w), false);
  auto full = conv2d(Variable(Tensor::fromVector({W, H, C, N}, x), false), wt, 2, 3, 3, 2)
                  .tensor().toHostVector();
  const size_t per = full.size() / N;
  for (int n = 0; n < N; ++n) {
    std::vector<float> xi(x.begin() + (size_t)n * C * H * W, x.begin() + (size_t)(n + 1) * C * H * W);
    auto one = conv2d(Variable(Tensor::fromVector({W, H, C, 1}, xi), false), wt, 2, 3, 3, 2)
                   .tensor().toHostVector();
    double worst = 0;
    for (size_t i = 0; i < per; ++i) worst = std::max(worst, (double)std::fabs(one[i] - full[n * per + i]));
    CHECK(worst <= 1e-5);
  }
}

// ModuleTest.cpp:177-194 (ConvPadding: SAME padding with strides and dilation),
// :382-396 (ConvolutionWithGroupFwd) and :398-413 (PoolingFwd): a batch equals its
// samples run one by one, with the reference's module arguments, sizes and tolerances
// Init.cpp:33-68: moments of the initialisers (the reference's InitTest checks shapes and types only)
static void testInit() {
  std::printf("initialisers\n");
  setSeed(11);
  const int fanIn = 576, n = 64 * 576;
  auto moments = [&](const Variable& v, double* mean, double* var, double* lo, double* hi) {
    const auto h = v.tensor().toHostVector();
    double s = 0, q = 0;
    *lo = 1e30; *hi = -1e30;
    for (float x : h) { s += x; q += (double)x * x; *lo = std::min<double>(*lo, x); *hi = std::max<double>(*hi, x); }
    *mean = s / h.size();
    *var = q / h.size() - *mean * *mean;
  };
  double m, v, lo, hi;
  moments(kaimingNormal(Shape({3, 3, 64, 64}), fanIn), &m, &v, &lo, &hi);
  CHECK(std::fabs(m) < 3e-4 && std::fabs(v * fanIn - 1.0) < 0.03);
  moments(kaimingUniform(Shape({3, 3, 64, 64}), fanIn), &m, &v, &lo, &hi);
  const double lim = std::sqrt(3.0 / fanIn);
  CHECK(std::fabs(m) < 3e-4 && std::fabs(v * fanIn - 1.0) < 0.03 && lo >= -lim && hi <= lim);
  moments(glorotNormal(Shape({n}), 100, 300), &m, &v, &lo, &hi);
  CHECK(std::fabs(v * 200 - 1.0) < 0.03);
  moments(glorotUniform(Shape({n}), 100, 300), &m, &v, &lo, &hi);
  CHECK(std::fabs(v * 200 - 1.0) < 0.03 && hi <= std::sqrt(3.0 / 200));
  CHECK(kaimingNormal(Shape({4, 4}), 16, dtype::bf16).type() == dtype::bf16);
}

static void testModuleShapesAndBatching() {
  std::printf("module shapes and batching\n");
  setSeed(5);
  {
    // written as in the reference: its `true, 1` land on the dilation arguments (1, 1)
    Conv2D conv1(30, 100, 3, 5, 2, 1, PaddingMode::SAME, 0, true, 1);
    Conv2D conv2(30, 100, 3, 5, 2, 1, PaddingMode::SAME, PaddingMode::SAME, true, 1);
    Conv2D conv3(30, 100, 10, 10, 1, 1, PaddingMode::SAME, PaddingMode::SAME, 4, 4);
    Variable input(Tensor::fromVector({32, 32, 30, 2}, randn((size_t)32 * 32 * 30 * 2, 41)), false);
    CHECK(conv1(input).shape() == Shape({16, 28, 100, 2}));
    CHECK(conv2(input).shape() == Shape({16, 32, 100, 2}));
    CHECK(conv3(input).shape() == Shape({32, 32, 100, 2}));
  }
  const int W = 120, H = 100, C = 30, N = 10;
  auto x = randn((size_t)N * C * H * W, 42);
  for (auto& v : x) v = 0.5f + 0.25f * v;
  auto batched = [&](Module& m, double tol, bool sameShape) {
    Variable in(Tensor::fromVector({W, H, C, N}, x), false);
    Variable out = m.forward({in}).front();
    if (sameShape) CHECK(out.shape() == in.shape());
    const std::vector<float> full = out.tensor().toHostVector();
    const size_t per = full.size() / N, pin = (size_t)C * H * W;
    for (int n = 0; n < N; ++n) {
      std::vector<float> xi(x.begin() + n * pin, x.begin() + (n + 1) * pin);
      const std::vector<float> one =
          m.forward({Variable(Tensor::fromVector({W, H, C, 1}, xi), false)}).front().tensor().toHostVector();
      double worst = one.size() == per ? 0 : 1e30;
      for (size_t i = 0; i < per && i < one.size(); ++i)
        worst = std::max(worst, (double)std::fabs(one[i] - full[n * per + i]));
      CHECK(worst <= tol);
    }
  };
  // as written in the reference, whose `true, 2` are dilation (1, 2), not bias and groups;
  // the grouped module follows
  Conv2D conv(30, 50, 9, 7, 2, 3, 3, 2, true, 2);
  batched(conv, 1e-5, false);
  Conv2D grouped(30, 50, 9, 7, 2, 3, 3, 2, 1, 1, true, 2);
  batched(grouped, 1e-5, false);
  Pool2D pool(9, 7, 1, 1, PaddingMode::SAME, PaddingMode::SAME);
  batched(pool, 1e-7, true);
}

static void testPool() {
  std::printf("pool2d\n");
  const int W = 12, H = 10, C = 3, N = 2;
  auto x = randn((size_t)N * C * H * W, 7);
  for (auto& v : x) v = std::round(v * 8.f) / 8.f;   // ties
  for (int mode = 0; mode < 3; ++mode) {
    flref_pool d{N, C, H, W, 3, 3, 2, 2, 1, 1, mode};
    int32_t OH, OW;
    flref_pool_out(&d, &OH, &OW);
    std::vector<float> y((size_t)N * C * OH * OW), dx(x.size());
    std::vector<uint8_t> am(y.size());
    auto dy = randn(y.size(), 8);
    flref_pool2d_fwd(&d, x.data(), y.data(), am.data());
    flref_pool2d_bwd(&d, dy.data(), am.data(), dx.data());
    Variable in(Tensor::fromVector({W, H, C, N}, x), true);
    Variable out = pool2d(in, 3, 3, 2, 2, 1, 1, (PoolingMode)mode);
    CHECK(out.shape() == Shape({OW, OH, C, N}));
    CHECK(out.tensor().toHostVector() == y);               // bit-exact
    out.backward(Variable(Tensor::fromVector(out.shape(), dy), false));
    CHECK(in.grad().tensor().toHostVector() == dx);        // bit-exact, tie routing included
  }
  // AutogradTest.cpp:333-337: 3x3x1x1 input, 2x2 window, stride 1
  Variable small(Tensor::fromVector({3, 3, 1, 1}, randn(9, 9)), true);
  CHECK(pool2d(small, 2, 2, 1, 1).shape() == Shape({2, 2, 1, 1}));
  // missing trailing dimensions count as 1 (onednn/Pool2D.cpp:95-98)
  Variable two(Tensor::fromVector({8, 6}, randn(48, 10)), false);
  CHECK(pool2d(two, 2, 2, 2, 2).shape() == Shape({4, 3, 1, 1}));
  // backward without the forward payload (onednn/Pool2D.cpp:190-193)
  AutogradExtension& e = getAutogradExtension(TensorBackendType::Hip);
  Tensor t({4, 4, 1, 1}, dtype::f32), g({2, 2, 1, 1}, dtype::f32);
  CHECK(throws<std::invalid_argument>(
      [&] { e.pool2dBackward(g, t, g, 2, 2, 2, 2, 0, 0, PoolingMode::MAX, nullptr); }));
  CHECK(throws<std::invalid_argument>([&] { pool2d(small, 2, 2, 1, 1, 2, 2); }));   // pad >= window
  // an operation that throws still pairs its begin with an abort: the profiler's depth returns to
  // zero, later operations get spans of their own and collect() finds every event recorded
  {
    StepProfiler prof;
    detail::setOpObserver(&prof);
    CHECK(throws<std::invalid_argument>(
        [&] { e.pool2dBackward(g, t, g, 2, 2, 2, 2, 0, 0, PoolingMode::MAX, nullptr); }));
    Variable again = pool2d(small, 2, 2, 1, 1);
    std::map<std::string, StepProfiler::Entry> got;
    CHECK(!throws<std::runtime_error>([&] { got = prof.collect(); }));
    CHECK(got["pool2dBackward"].calls == 1 && got["pool2d"].calls == 1);
    detail::setOpObserver(nullptr);
  }
}

static void testBatchnorm() {
  std::printf("batchnorm\n");
  const int W = 13, H = 13, C = 3, N = 8;
  auto x = randn((size_t)N * C * H * W, 11, 1.4f, 0.5f), g = randn(C, 12, 0.1f, 1.f), b = randn(C, 13);
  auto dy = randn(x.size(), 14);
  std::vector<float> y(x.size()), mean(C), var(C), dx(x.size()), dg(C), db(C);
  flref_bn_fwd_train(N, C, (int64_t)H * W, x.data(), g.data(), b.data(), 1e-5, y.data(), mean.data(), var.data());
  flref_bn_bwd(N, C, (int64_t)H * W, x.data(), dy.data(), g.data(), mean.data(), var.data(), 1e-5,
               dx.data(), dg.data(), db.data());
  Variable in(Tensor::fromVector({W, H, C, N}, x), true);
  Variable wt(Tensor::fromVector({C}, g), true), bs(Tensor::fromVector({C}, b), true);
  Variable rm, rv;   // empty: created by the op (onednn/BatchNorm.cpp:116-122)
  Variable out = batchnorm(in, wt, bs, rm, rv, {2}, true, 0.0, 1e-5);
  CHECK(relL2(out.tensor().toHostVector(), y) <= 1e-4);
  // momentum 0: running buffers hold the batch statistics (onednn/BatchNorm.cpp:154-157)
  CHECK(relL2(rm.tensor().toHostVector(), mean) <= 1e-5);
  CHECK(relL2(rv.tensor().toHostVector(), var) <= 1e-4);
  out.backward(Variable(Tensor::fromVector(out.shape(), dy), false));
  CHECK(relL2(in.grad().tensor().toHostVector(), dx) <= 1e-4);
  CHECK(relL2(wt.grad().tensor().toHostVector(), dg) <= 1e-4);
  CHECK(relL2(bs.grad().tensor().toHostVector(), db) <= 1e-4);

  // momentum 0.1: r = 0.9 r + 0.1 batch with the unbiased variance
  Variable rm2(Tensor::full({C}, 0., dtype::f32), false), rv2(Tensor::full({C}, 1., dtype::f32), false);
  batchnorm(in, wt, bs, rm2, rv2, {2}, true, 0.1, 1e-5);
  std::vector<float> erm(C, 0.f), erv(C, 1.f);
  flref_bn_running_update(C, (int64_t)N * H * W, mean.data(), var.data(), 0.1, erm.data(), erv.data());
  CHECK(relL2(rm2.tensor().toHostVector(), erm) <= 1e-5);
  CHECK(relL2(rv2.tensor().toHostVector(), erv) <= 1e-4);

  // inference with running statistics, with and without affine parameters
  std::vector<float> yi(x.size());
  flref_bn_fwd_infer(N, C, (int64_t)H * W, x.data(), g.data(), b.data(), erm.data(), erv.data(), 1e-5, yi.data());
  Variable nograd(in.tensor(), false);
  Variable wng(wt.tensor(), false), bng(bs.tensor(), false);
  CHECK(relL2(batchnorm(nograd, wng, bng, rm2, rv2, {2}, false, 0.0, 1e-5).tensor().toHostVector(), yi) <= 1e-5);
  flref_bn_fwd_infer(N, C, (int64_t)H * W, x.data(), nullptr, nullptr, erm.data(), erv.data(), 1e-5, yi.data());
  Variable none1, none2;
  CHECK(relL2(batchnorm(nograd, none1, none2, rm2, rv2, {2}, false, 0.0, 1e-5).tensor().toHostVector(), yi) <= 1e-5);

  // per-activation mode, axes {0,1,2} (AutogradNormalizationTest.cpp:191-226)
  const int64_t nf = (int64_t)W * H * C;
  auto g3 = randn(nf, 15, 0.1f, 1.f), b3 = randn(nf, 16);
  std::vector<float> y3(x.size()), m3(nf), v3(nf);
  flref_bn_fwd_train(N, nf, 1, x.data(), g3.data(), b3.data(), 1e-5, y3.data(), m3.data(), v3.data());
  Variable w3(Tensor::fromVector({(Dim)nf}, g3), false), bb3(Tensor::fromVector({(Dim)nf}, b3), false);
  Variable rm3, rv3;
  CHECK(relL2(batchnorm(nograd, w3, bb3, rm3, rv3, {0, 1, 2}, true, 0.0, 1e-5).tensor().toHostVector(), y3) <= 1e-4);

  // errors: non-contiguous axes (onednn/BatchNorm.cpp:124-130), mixed types, missing payload
  CHECK(throws<std::invalid_argument>([&] { batchnorm(nograd, none1, none2, rm3, rv3, {0, 2}, true, 0.0, 1e-5); }));
  Variable wbf(wt.tensor().astype(dtype::bf16), false);
  CHECK(throws<std::invalid_argument>([&] { batchnorm(nograd, wbf, none2, rm2, rv2, {2}, true, 0.0, 1e-5); }));
  AutogradExtension& e = getAutogradExtension(TensorBackendType::Hip);
  Tensor empty;
  CHECK(throws<std::invalid_argument>(
      [&] { e.batchnormBackward(in.tensor(), empty, empty, in.tensor(), wt.tensor(), {2}, true, 1e-5f, nullptr); }));
}

static void testGradAccumulation() {
  std::printf("gradient accumulation\n");
  // one input feeding two pools: the gradients add (Variable.cpp:185-218)
  const int W = 8, H = 8;
  auto x = randn(64, 17);
  Variable in(Tensor::fromVector({W, H, 1, 1}, x), true);
  Variable a = pool2d(in, 2, 2, 2, 2, 0, 0, PoolingMode::AVG_INCLUDE_PADDING);
  std::vector<float> ones(16, 1.f);
  a.backward(Variable(Tensor::fromVector(a.shape(), ones), false));
  Variable b = pool2d(in, 2, 2, 2, 2, 0, 0, PoolingMode::AVG_INCLUDE_PADDING);
  b.backward(Variable(Tensor::fromVector(b.shape(), ones), false));
  auto g = in.grad().tensor().toHostVector();
  bool ok = true;
  for (float v : g) ok = ok && v == 0.5f;
  CHECK(ok);
}

static std::vector<float> uniformv(size_t n, unsigned seed, float bound) {
  std::mt19937 gen(seed);
  std::uniform_real_distribution<float> d(-bound, bound);
  std::vector<float> v(n);
  for (auto& x : v) x = d(gen);
  return v;
}

// One forward + backward step of the README convnet (README.md:45-84; dropout left out):
// View, Conv2D 1->32 5x5 SAME, ReLU, Pool2D 2x2 s2, Conv2D 32->64 5x5 SAME, ReLU, Pool2D,
// View, Linear 3136->1024, ReLU, Linear 1024->10, LogSoftmax, categoricalCrossEntropy;
// loss.backward() through the tape against the CPU checker run layer by layer.
static void testMnistStep() {
  std::printf("MNIST convnet training step\n");
  const int B = 8;
  auto x = randn((size_t)B * 28 * 28, 21);
  std::vector<int32_t> labels(B);
  for (int i = 0; i < B; ++i) labels[i] = (i * 7 + 3) % 10;
  // Conv2D::initialize / Linear::initialize: Kaiming-uniform weights, bias U(+-sqrt(1/fanIn))
  auto w1 = uniformv(32 * 25, 22, std::sqrt(3.f / 25)), b1 = uniformv(32, 23, std::sqrt(1.f / 25));
  auto w2 = uniformv(64 * 32 * 25, 24, std::sqrt(3.f / 800)), b2 = uniformv(64, 25, std::sqrt(1.f / 800));
  auto w3 = uniformv((size_t)1024 * 3136, 26, std::sqrt(3.f / 3136)), b3 = uniformv(1024, 27, std::sqrt(1.f / 3136));
  auto w4 = uniformv(10 * 1024, 28, std::sqrt(3.f / 1024)), b4 = uniformv(10, 29, std::sqrt(1.f / 1024));
  const int pad = derivePadding(28, 5, 1, -1, 1);
  CHECK(pad == 2);

  // ---- CPU checker ---------------------------------------------------------------
  flref_conv d1{B, 1, 28, 28, 32, 5, 5, 1, 1, pad, pad, 1, 1, 1}, d2{B, 32, 14, 14, 64, 5, 5, 1, 1, pad, pad, 1, 1, 1};
  flref_pool p1{B, 32, 28, 28, 2, 2, 2, 2, 0, 0, 0}, p2{B, 64, 14, 14, 2, 2, 2, 2, 0, 0, 0};
  std::vector<float> a1((size_t)B * 32 * 784), r1(a1.size()), q1((size_t)B * 32 * 196);
  std::vector<uint8_t> m1(q1.size());
  std::vector<float> a2((size_t)B * 64 * 196), r2(a2.size()), q2((size_t)B * 64 * 49);
  std::vector<uint8_t> m2(q2.size());
  std::vector<float> a3((size_t)B * 1024), r3(a3.size()), a4((size_t)B * 10), lp(a4.size());
  flref_conv2d_fwd(&d1, x.data(), w1.data(), b1.data(), a1.data());
  flref_relu_fwd((int64_t)a1.size(), a1.data(), r1.data());
  flref_pool2d_fwd(&p1, r1.data(), q1.data(), m1.data());
  flref_conv2d_fwd(&d2, q1.data(), w2.data(), b2.data(), a2.data());
  flref_relu_fwd((int64_t)a2.size(), a2.data(), r2.data());
  flref_pool2d_fwd(&p2, r2.data(), q2.data(), m2.data());
  flref_matmul(1024, B, 3136, 0, 0, w3.data(), q2.data(), b3.data(), a3.data());
  flref_relu_fwd((int64_t)a3.size(), a3.data(), r3.data());
  flref_matmul(10, B, 1024, 0, 0, w4.data(), r3.data(), b4.data(), a4.data());
  flref_logsoftmax_fwd(10, B, a4.data(), lp.data());
  float loss[2], count;
  CHECK(flref_cce_fwd(10, B, lp.data(), labels.data(), -1, nullptr, loss, &count) == 0);
  const float one = 1.f;
  std::vector<float> g4(a4.size()), g4b(a4.size()), dw4(w4.size()), db4(10), g3(a3.size()), dw3(w3.size()), db3(1024);
  std::vector<float> gq2(q2.size()), gr2(r2.size()), dw2(w2.size()), db2(64), gq1(q1.size()), gr1(r1.size()), dw1(w1.size()), db1(32);
  flref_cce_bwd(10, B, &one, labels.data(), -1, 1, count, g4.data());
  flref_logsoftmax_bwd(10, B, g4.data(), lp.data(), g4b.data());
  flref_sum_columns(10, B, g4b.data(), db4.data());
  flref_matmul(10, 1024, B, 0, 1, g4b.data(), r3.data(), nullptr, dw4.data());
  flref_matmul(1024, B, 10, 1, 0, w4.data(), g4b.data(), nullptr, g3.data());
  flref_relu_bwd((int64_t)g3.size(), g3.data(), a3.data(), g3.data());
  flref_sum_columns(1024, B, g3.data(), db3.data());
  flref_matmul(1024, 3136, B, 0, 1, g3.data(), q2.data(), nullptr, dw3.data());
  flref_matmul(3136, B, 1024, 1, 0, w3.data(), g3.data(), nullptr, gq2.data());
  flref_pool2d_bwd(&p2, gq2.data(), m2.data(), gr2.data());
  flref_relu_bwd((int64_t)gr2.size(), gr2.data(), a2.data(), gr2.data());
  flref_conv2d_bwd_filter(&d2, q1.data(), gr2.data(), dw2.data(), db2.data());
  flref_conv2d_bwd_data(&d2, gr2.data(), w2.data(), gq1.data());
  flref_pool2d_bwd(&p1, gq1.data(), m1.data(), gr1.data());
  flref_relu_bwd((int64_t)gr1.size(), gr1.data(), a1.data(), gr1.data());
  flref_conv2d_bwd_filter(&d1, x.data(), gr1.data(), dw1.data(), db1.data());

  // ---- device, through the tape ---------------------------------------------------
  Variable in(Tensor::fromVector({28 * 28, B}, x), false);
  Variable W1(Tensor::fromVector({5, 5, 1, 32}, w1), true), B1(Tensor::fromVector({1, 1, 32, 1}, b1), true);
  Variable W2(Tensor::fromVector({5, 5, 32, 64}, w2), true), B2(Tensor::fromVector({1, 1, 64, 1}, b2), true);
  Variable W3(Tensor::fromVector({1024, 3136}, w3), true), B3(Tensor::fromVector({1024}, b3), true);
  Variable W4(Tensor::fromVector({10, 1024}, w4), true), B4(Tensor::fromVector({10}, b4), true);
  Variable tg(Tensor::fromHost(Shape({B}), dtype::s32, labels.data()), false);
  Variable h = moddims(in, Shape({28, 28, 1, -1}));
  h = pool2d(relu(conv2d(h, W1, B1, 1, 1, pad, pad)), 2, 2, 2, 2);
  h = pool2d(relu(conv2d(h, W2, B2, 1, 1, pad, pad)), 2, 2, 2, 2);
  CHECK(h.shape() == Shape({7, 7, 64, B}));
  h = moddims(h, Shape({7 * 7 * 64, -1}));
  h = relu(linear(h, W3, B3));
  Variable out = logSoftmax(linear(h, W4, B4), 0);
  CHECK(out.shape() == Shape({10, B}));
  CHECK(relL2(out.tensor().toHostVector(), lp) <= 1e-4);
  Variable L = categoricalCrossEntropy(out, tg);
  CHECK(std::fabs(L.tensor().toHostVector()[0] - loss[1]) <= 1e-5f * std::max(1.f, std::fabs(loss[1])));
  L.backward(Variable(Tensor::fromVector({1}, {1.f}), false));
  CHECK(relL2(W4.grad().tensor().toHostVector(), dw4) <= 1e-4 && relL2(B4.grad().tensor().toHostVector(), db4) <= 1e-4);
  CHECK(relL2(W3.grad().tensor().toHostVector(), dw3) <= 1e-4 && relL2(B3.grad().tensor().toHostVector(), db3) <= 1e-4);
  CHECK(relL2(W2.grad().tensor().toHostVector(), dw2) <= 1e-4 && relL2(B2.grad().tensor().toHostVector(), db2) <= 1e-4);
  CHECK(relL2(W1.grad().tensor().toHostVector(), dw1) <= 1e-4 && relL2(B1.grad().tensor().toHostVector(), db1) <= 1e-4);
  CHECK(!in.isCalcGrad());
  // targets outside [0, classes) throw like the reference (Functions.cpp:1100-1108)
  std::vector<int32_t> badl(B, 10);
  Variable bad(Tensor::fromHost(Shape({B}), dtype::s32, badl.data()), false);
  CHECK(throws<std::invalid_argument>([&] { categoricalCrossEntropy(out, bad); }));
  CHECK(throws<std::invalid_argument>([&] { moddims(in, Shape({5, -1})); }));
}

static std::vector<float> hostOf(const Variable& v) { return v.tensor().toHostVector(); }

// The README network built from modules: same result as the functional chain on the
// modules' own parameters, initialisation bounds, train/eval, zeroGrad, setParams.
static void testSequentialMnist() {
  std::printf("Sequential MNIST convnet\n");
  const int B = 4;
  setSeed(5);
  Sequential model;
  model.add(View(Shape({28, 28, 1, -1})));
  model.add(Conv2D(1, 32, 5, 5, 1, 1, PaddingMode::SAME, PaddingMode::SAME));
  model.add(ReLU());
  model.add(Pool2D(2, 2, 2, 2));
  model.add(Conv2D(32, 64, 5, 5, 1, 1, PaddingMode::SAME, PaddingMode::SAME));
  model.add(ReLU());
  model.add(Pool2D(2, 2, 2, 2));
  model.add(View(Shape({7 * 7 * 64, -1})));
  model.add(Linear(7 * 7 * 64, 1024));
  model.add(ReLU());
  model.add(Linear(1024, 10));
  model.add(LogSoftmax());
  CHECK(model.params().size() == 8 && model.modules().size() == 12);
  CHECK(model.param(0).shape() == Shape({5, 5, 1, 32}) && model.param(1).shape() == Shape({1, 1, 32, 1}));
  CHECK(model.param(4).shape() == Shape({1024, 3136}) && model.param(7).shape() == Shape({10}));
  // Kaiming-uniform bounds: sqrt(3 / fanIn) for weights, sqrt(1 / fanIn) for biases
  const double lim[8] = {std::sqrt(3. / 25), std::sqrt(1. / 25), std::sqrt(3. / 800), std::sqrt(1. / 800),
                         std::sqrt(3. / 3136), std::sqrt(1. / 3136), std::sqrt(3. / 1024), std::sqrt(1. / 1024)};
  for (int i = 0; i < 8; ++i) {
    const auto v = hostOf(model.param(i));
    float mx = 0.f;
    double mean = 0;
    for (float f : v) {
      mx = std::max(mx, std::fabs(f));
      mean += f;
    }
    CHECK(mx <= lim[i] * 1.0000001 && mx >= (v.size() >= 32 ? 0.8 : 0.3) * lim[i]);
    if (v.size() > 10000) CHECK(std::fabs(mean / v.size()) < 0.02 * lim[i]);
  }
  CHECK(model.prettyString().find("Conv2D (32->64, 5x5, 1,1, SAME,SAME, 1, 1) (with bias)") != std::string::npos);

  auto x = randn((size_t)B * 28 * 28, 31);
  std::vector<int32_t> labels = {3, 1, 4, 1};
  Variable in(Tensor::fromVector({28 * 28, B}, x), false);
  Variable tg(Tensor::fromHost(Shape({B}), dtype::s32, labels.data()), false);
  Variable out = model.forward(in);
  CHECK(out.shape() == Shape({10, B}));
  // the functional chain on the same parameters
  auto P = model.params();
  Variable h = moddims(in, Shape({28, 28, 1, -1}));
  h = pool2d(relu(conv2d(h, P[0], P[1], 1, 1, 2, 2)), 2, 2, 2, 2);
  h = pool2d(relu(conv2d(h, P[2], P[3], 1, 1, 2, 2)), 2, 2, 2, 2);
  h = relu(linear(moddims(h, Shape({7 * 7 * 64, -1})), P[4], P[5]));
  Variable ref = logSoftmax(linear(h, P[6], P[7]), 0);
  CHECK(hostOf(out) == hostOf(ref));
  CategoricalCrossEntropy criterion;
  Variable loss = criterion(out, tg);
  loss.backward(Variable(Tensor::fromVector({1}, {1.f}), false));
  std::vector<std::vector<float>> grads;
  for (auto& p : model.params()) {
    CHECK(p.isGradAvailable());
    grads.push_back(hostOf(p.grad()));
  }
  model.zeroGrad();
  for (auto& p : model.params()) CHECK(!p.isGradAvailable());
  Variable loss2 = categoricalCrossEntropy(ref, tg);
  loss2.backward(Variable(Tensor::fromVector({1}, {1.f}), false));
  for (int i = 0; i < 8; ++i) CHECK(hostOf(model.param(i).grad()) == grads[i]);
  CHECK(hostOf(loss) == hostOf(loss2));

  // eval(): parameters stop asking for gradients, in the children as well (Module.cpp:58-70)
  model.eval();
  CHECK(!model.isTrain() && !model.module(1)->isTrain());
  for (auto& p : model.params()) CHECK(!p.isCalcGrad());
  CHECK(!model.forward(in).isCalcGrad());
  model.train();
  for (auto& p : model.params()) CHECK(p.isCalcGrad());
  // setParams reaches the child module (Container.cpp:85-93)
  Variable zeroBias(Tensor::full({10}, 0., dtype::f32), true);
  model.setParams(zeroBias, 7);
  CHECK(hostOf(model.module(10)->param(1)) == std::vector<float>(10, 0.f));
  CHECK(throws<std::out_of_range>([&] { model.param(8); }));
  CHECK(throws<std::invalid_argument>([&] { model.forward(std::vector<Variable>{in, in}); }));
  // bias shape rules of Conv2D(w, b) (Conv2D.cpp:88-96)
  Variable w(Tensor::full({3, 3, 4, 6}, 0.1, dtype::f32), true), bad(Tensor::full({1, 1, 5, 1}, 0., dtype::f32), true);
  CHECK(throws<std::invalid_argument>([&] { Conv2D(w, bad); }));
}

// BatchNorm module: exponential and cumulative running statistics over several
// batches, eval mode, statistics not tracked (BatchNorm.cpp:74-112)
static void testBatchNormModule() {
  std::printf("BatchNorm module\n");
  const int W = 6, H = 5, C = 4, N = 7;
  const int64_t M = (int64_t)N * H * W;
  setSeed(9);
  BatchNorm bn(2, C), cum(2, C, -1.0), loose(2, C, 0.1, 1e-5, true, false);
  CHECK(hostOf(bn.runningMean()) == std::vector<float>(C, 0.f) && hostOf(bn.runningVar()) == std::vector<float>(C, 1.f));
  CHECK(hostOf(bn.param(1)) == std::vector<float>(C, 0.f));
  for (float f : hostOf(bn.param(0))) CHECK(f >= 0.f && f <= 1.f);
  std::vector<float> erm(C, 0.f), erv(C, 1.f), crm(C, 0.f), crv(C, 1.f);
  std::vector<float> x, y(x.size()), mean(C), var(C);
  const auto g = hostOf(bn.param(0)), b = hostOf(bn.param(1));
  const auto gc = hostOf(cum.param(0)), bc = hostOf(cum.param(1));
  for (int step = 1; step <= 3; ++step) {
    x = randn((size_t)N * C * H * W, 40 + step, 1.f + 0.3f * step, 0.2f * step);
    y.resize(x.size());
    flref_bn_fwd_train(N, C, (int64_t)H * W, x.data(), g.data(), b.data(), 1e-5, y.data(), mean.data(), var.data());
    flref_bn_running_update(C, M, mean.data(), var.data(), 0.1, erm.data(), erv.data());
    flref_bn_running_update(C, M, mean.data(), var.data(), 1.0 / step, crm.data(), crv.data());
    Variable in(Tensor::fromVector({W, H, C, N}, x), true);
    CHECK(relL2(hostOf(bn.forward(in)), y) <= 1e-4);
    cum.forward(in);
    CHECK(bn.numBatchesTracked() == step);
  }
  CHECK(relL2(hostOf(bn.runningMean()), erm) <= 1e-5 && relL2(hostOf(bn.runningVar()), erv) <= 1e-4);
  // momentum < 0: the running mean is the plain average of the batch means
  CHECK(relL2(hostOf(cum.runningMean()), crm) <= 1e-5 && relL2(hostOf(cum.runningVar()), crv) <= 1e-4);
  // eval: running statistics, no update, no gradient request
  bn.eval();
  Variable in(Tensor::fromVector({W, H, C, N}, x), false);
  flref_bn_fwd_infer(N, C, (int64_t)H * W, x.data(), g.data(), b.data(), erm.data(), erv.data(), 1e-5, y.data());
  Variable ye = bn.forward(in);
  CHECK(relL2(hostOf(ye), y) <= 1e-5 && !ye.isCalcGrad() && bn.numBatchesTracked() == 3);
  CHECK(relL2(hostOf(bn.runningMean()), erm) <= 1e-5);
  // statistics not tracked: batch statistics also in eval mode
  const auto gl = hostOf(loose.param(0)), bl = hostOf(loose.param(1));
  loose.eval();
  flref_bn_fwd_train(N, C, (int64_t)H * W, x.data(), gl.data(), bl.data(), 1e-5, y.data(), mean.data(), var.data());
  CHECK(relL2(hostOf(loose.forward(in)), y) <= 1e-4 && loose.numBatchesTracked() == 0);
  // a 16-bit input keeps f32 parameters (BatchNorm.cpp:86-88: half input)
  bn.train();
  for (const dtype lo : {dtype::bf16, dtype::f16}) {
    Variable in16(in.tensor().astype(lo), true);
    Variable y16 = bn.forward(in16);
    CHECK(y16.type() == lo);
    y16.backward(Variable(Tensor::full(y16.shape(), 1., dtype::f32).astype(lo), false));
    CHECK(bn.param(0).grad().type() == dtype::f32 && in16.grad().type() == lo);
  }
}

// LayerNorm module on the reference test's shapes (ModuleTest.cpp:670-719) plus the
// transformer use (normalise dimension 0 of [C, T, B]) with per-element parameters
static void testLayerNormModule() {
  std::printf("LayerNorm module\n");
  const double eps = 1e-5;
  const int F = 10, S = 4 * 4 * 3;
  auto x = randn((size_t)S * F, 51, 1.f, 0.5f);
  Variable input(Tensor::fromVector({4, 4, 3, F}, x), true);
  // direct definition: mean and biased variance over axis 3
  std::vector<float> want(x.size());
  for (int s = 0; s < S; ++s) {
    double m = 0, v = 0;
    for (int f = 0; f < F; ++f) m += x[(size_t)f * S + s];
    m /= F;
    for (int f = 0; f < F; ++f) v += (x[(size_t)f * S + s] - m) * (x[(size_t)f * S + s] - m);
    v /= F;
    for (int f = 0; f < F; ++f) want[(size_t)f * S + s] = (float)((x[(size_t)f * S + s] - m) / std::sqrt(v + eps));
  }
  LayerNorm module1(std::vector<int>{3}, eps, false);
  module1.train();
  Variable out = module1.forward(input);
  CHECK(relL2(hostOf(out), want) <= 1e-4 && out.type() == input.type());
  module1.eval();
  CHECK(relL2(hostOf(module1.forward(input)), want) <= 1e-4);
  LayerNorm module2(std::vector<int>{3}, eps, true);
  module2.train();
  const auto outTrain = hostOf(module2.forward(input));
  module2.eval();
  CHECK(hostOf(module2.forward(input)) == outTrain && relL2(outTrain, want) <= 1e-4);
  LayerNorm module3(std::vector<int>{3}, eps, true, F);
  module3.setParams(Variable(Tensor::full({F}, 1.0, dtype::f32), false), 0);
  module3.setParams(Variable(Tensor::full({F}, 0.0, dtype::f32), false), 1);
  CHECK(relL2(hostOf(module3.forward(input)), outTrain) <= 1e-6);
  Variable input3(Tensor::fromVector({4, 4, 3}, randn(48, 52)), true);
  LayerNorm module4(std::vector<int>{0}, eps, false);
  CHECK(module4.forward(input3).shape() == input3.shape());
  // a complement that is not contiguous goes through fl::reorder (LayerNorm.cpp:63-86): normalise
  // over dimensions {0, 2} of [4, 4, 3, F], i.e. per (h, n) over (w, c); direct definition
  {
    LayerNorm module5(std::vector<int>{0, 2}, eps, false);
    std::vector<float> want5(x.size());
    for (int n = 0; n < F; ++n)
      for (int h = 0; h < 4; ++h) {
        auto at = [&](int w_, int c) { return ((size_t)(n * 3 + c) * 4 + h) * 4 + w_; };
        double m = 0, v = 0;
        for (int c = 0; c < 3; ++c) for (int w_ = 0; w_ < 4; ++w_) m += x[at(w_, c)];
        m /= 12;
        for (int c = 0; c < 3; ++c) for (int w_ = 0; w_ < 4; ++w_) v += (x[at(w_, c)] - m) * (x[at(w_, c)] - m);
        v /= 12;
        for (int c = 0; c < 3; ++c) for (int w_ = 0; w_ < 4; ++w_) want5[at(w_, c)] = (float)((x[at(w_, c)] - m) / std::sqrt(v + eps));
      }
    Variable out5 = module5.forward(input);
    CHECK(out5.shape() == input.shape() && relL2(hostOf(out5), want5) <= 1e-4);
  }
  // normalise dimension 1 of [W, H, C, N] with one scale / shift element per h (complement {0, 2, 3}):
  // equals the contiguous case on the tensor transposed by hand to [H, W, C, N], outputs and gradients
  {
    const int W_ = 6, H_ = 5, C_ = 3, N_ = 4;
    auto xa = randn((size_t)W_ * H_ * C_ * N_, 57, 1.5f, 0.2f), dya = randn(xa.size(), 58);
    auto wa = randn(H_, 59, 0.3f, 1.f), ba = randn(H_, 60);
    std::vector<float> xb(xa.size()), dyb(xa.size());
    auto ia = [&](int w_, int h, int r) { return ((size_t)r * H_ + h) * W_ + w_; };   // r = (n, c) flattened
    auto ib = [&](int w_, int h, int r) { return ((size_t)r * W_ + w_) * H_ + h; };
    for (int r = 0; r < C_ * N_; ++r)
      for (int h = 0; h < H_; ++h)
        for (int w_ = 0; w_ < W_; ++w_) { xb[ib(w_, h, r)] = xa[ia(w_, h, r)]; dyb[ib(w_, h, r)] = dya[ia(w_, h, r)]; }
    LayerNorm lnA(1, eps, true, H_), lnB(0, eps, true, H_);
    for (LayerNorm* m : {&lnA, &lnB}) {
      m->setParams(Variable(Tensor::fromVector({H_}, wa), true), 0);
      m->setParams(Variable(Tensor::fromVector({H_}, ba), true), 1);
    }
    Variable va(Tensor::fromVector({W_, H_, C_, N_}, xa), true), vb(Tensor::fromVector({H_, W_, C_, N_}, xb), true);
    Variable oa = lnA.forward(va), ob = lnB.forward(vb);
    oa.backward(Variable(Tensor::fromVector({W_, H_, C_, N_}, dya), false));
    ob.backward(Variable(Tensor::fromVector({H_, W_, C_, N_}, dyb), false));
    auto unperm = [&](const std::vector<float>& b_) {
      std::vector<float> a_(b_.size());
      for (int r = 0; r < C_ * N_; ++r)
        for (int h = 0; h < H_; ++h)
          for (int w_ = 0; w_ < W_; ++w_) a_[ia(w_, h, r)] = b_[ib(w_, h, r)];
      return a_;
    };
    CHECK(oa.shape() == Shape({W_, H_, C_, N_}));
    CHECK(relL2(hostOf(oa), unperm(hostOf(ob))) <= 1e-6);
    CHECK(relL2(hostOf(va.grad()), unperm(hostOf(vb.grad()))) <= 1e-6);
    CHECK(relL2(hostOf(lnA.param(0).grad()), hostOf(lnB.param(0).grad())) <= 1e-6);
    CHECK(relL2(hostOf(lnA.param(1).grad()), hostOf(lnB.param(1).grad())) <= 1e-6);
    // fl::reorder itself: the inverse permutation restores the tensor bit for bit
    Variable rr = reorder(reorder(va, Shape({2, 0, 3, 1})), Shape({1, 3, 0, 2}));
    CHECK(hostOf(rr) == xa);
    CHECK(throws<std::invalid_argument>([&] { reorder(va, Shape({0, 0, 1, 2})); }));
  }
  CHECK(throws<std::invalid_argument>([&] { LayerNorm(std::vector<int>{3}, eps, true, F + 1).forward(input); }));

  // [C, T, B], normalise C with per-element scale and shift; forward and backward against
  // the CPU checker (batchnorm over the complement, then the broadcast affine)
  const int Cn = 24, T = 9, Bn = 5;
  auto xt = randn((size_t)Cn * T * Bn, 53, 2.f, -0.3f), dyt = randn(xt.size(), 54);
  auto w = randn(Cn, 55, 0.2f, 1.f), b = randn(Cn, 56);
  std::vector<float> ones(T * Bn, 1.f), zeros(T * Bn, 0.f), xhat(xt.size()), mean(T * Bn), var(T * Bn), y(xt.size());
  flref_bn_fwd_train(1, T * Bn, Cn, xt.data(), ones.data(), zeros.data(), eps, xhat.data(), mean.data(), var.data());
  flref_affine_fwd(T * Bn, Cn, 1, 0, xhat.data(), w.data(), b.data(), y.data());
  std::vector<float> g(xt.size()), dw(Cn), db(Cn), dx(xt.size()), dgam(T * Bn), dbet(T * Bn);
  flref_affine_bwd(T * Bn, Cn, 1, 0, dyt.data(), xhat.data(), w.data(), g.data(), dw.data(), db.data());
  flref_bn_bwd(1, T * Bn, Cn, xt.data(), g.data(), ones.data(), mean.data(), var.data(), eps, dx.data(),
               dgam.data(), dbet.data());
  LayerNorm ln(0, eps, true, Cn);
  ln.setParams(Variable(Tensor::fromVector({Cn}, w), true), 0);
  ln.setParams(Variable(Tensor::fromVector({Cn}, b), true), 1);
  Variable vin(Tensor::fromVector({Cn, T, Bn}, xt), true);
  Variable vout = ln.forward(vin);
  CHECK(vout.shape() == Shape({Cn, T, Bn}) && relL2(hostOf(vout), y) <= 1e-4);
  vout.backward(Variable(Tensor::fromVector({Cn, T, Bn}, dyt), false));
  CHECK(relL2(hostOf(vin.grad()), dx) <= 1e-4);
  CHECK(relL2(hostOf(ln.param(0).grad()), dw) <= 1e-4 && relL2(hostOf(ln.param(1).grad()), db) <= 1e-4);
}

// One ResNet bottleneck (pkg/vision/models/Resnet.cpp:38-87: 1x1 -> 3x3 -> 1x1, BatchNorm
// after every convolution, ReLU, residual add, ReLU) from modules, forward and backward
// against the CPU checker
static void testBottleneck() {
  std::printf("ResNet bottleneck from modules\n");
  const int W = 14, H = 14, Cin = 16, Cm = 8, N = 4;
  const int64_t HW = (int64_t)H * W;
  setSeed(13);
  Conv2D c1(Cin, Cm, 1, 1, 1, 1, 0, 0, 1, 1, false), c2(Cm, Cm, 3, 3, 1, 1, PaddingMode::SAME, PaddingMode::SAME, 1, 1, false),
      c3(Cm, Cin, 1, 1, 1, 1, 0, 0, 1, 1, false);
  BatchNorm b1(2, Cm), b2(2, Cm), b3(2, Cin);
  auto x = randn((size_t)N * Cin * HW, 61), dy = randn((size_t)N * Cin * HW, 62);
  Variable in(Tensor::fromVector({W, H, Cin, N}, x), true);
  Variable t3 = b3(c3(relu(b2(c2(relu(b1(c1(in))))))));
  Variable out = relu(t3 + in);
  out.backward(Variable(Tensor::fromVector(out.shape(), dy), false));

  // ---- CPU checker -------------------------------------------------------------------
  const auto w1 = hostOf(c1.param(0)), w2 = hostOf(c2.param(0)), w3 = hostOf(c3.param(0));
  const auto g1 = hostOf(b1.param(0)), g2 = hostOf(b2.param(0)), g3 = hostOf(b3.param(0));
  const auto z1 = hostOf(b1.param(1)), z2 = hostOf(b2.param(1)), z3 = hostOf(b3.param(1));
  flref_conv d1{N, Cin, H, W, Cm, 1, 1, 1, 1, 0, 0, 1, 1, 1}, d2{N, Cm, H, W, Cm, 3, 3, 1, 1, 1, 1, 1, 1, 1},
      d3{N, Cm, H, W, Cin, 1, 1, 1, 1, 0, 0, 1, 1, 1};
  const size_t nm = (size_t)N * Cm * HW, ni = (size_t)N * Cin * HW;
  std::vector<float> a1(nm), n1(nm), r1(nm), a2(nm), n2(nm), r2(nm), a3(ni), n3(ni), s(ni), o(ni);
  std::vector<float> m1(Cm), v1(Cm), m2(Cm), v2(Cm), m3(Cin), v3(Cin);
  flref_conv2d_fwd(&d1, x.data(), w1.data(), nullptr, a1.data());
  flref_bn_fwd_train(N, Cm, HW, a1.data(), g1.data(), z1.data(), 1e-5, n1.data(), m1.data(), v1.data());
  flref_relu_fwd((int64_t)nm, n1.data(), r1.data());
  flref_conv2d_fwd(&d2, r1.data(), w2.data(), nullptr, a2.data());
  flref_bn_fwd_train(N, Cm, HW, a2.data(), g2.data(), z2.data(), 1e-5, n2.data(), m2.data(), v2.data());
  flref_relu_fwd((int64_t)nm, n2.data(), r2.data());
  flref_conv2d_fwd(&d3, r2.data(), w3.data(), nullptr, a3.data());
  flref_bn_fwd_train(N, Cin, HW, a3.data(), g3.data(), z3.data(), 1e-5, n3.data(), m3.data(), v3.data());
  for (size_t i = 0; i < ni; ++i) s[i] = n3[i] + x[i];
  flref_relu_fwd((int64_t)ni, s.data(), o.data());
  CHECK(relL2(hostOf(out), o) <= 1e-4);
  std::vector<float> gs(ni), ga3(ni), dg3(Cin), db3(Cin), gr2(nm), dw3(w3.size()), gn2(nm), ga2(nm), dg2(Cm), db2(Cm),
      gr1(nm), dw2(w2.size()), gn1(nm), ga1(nm), dg1(Cm), db1(Cm), gx(ni), dw1(w1.size());
  flref_relu_bwd((int64_t)ni, dy.data(), s.data(), gs.data());
  flref_bn_bwd(N, Cin, HW, a3.data(), gs.data(), g3.data(), m3.data(), v3.data(), 1e-5, ga3.data(), dg3.data(), db3.data());
  flref_conv2d_bwd_filter(&d3, r2.data(), ga3.data(), dw3.data(), nullptr);
  flref_conv2d_bwd_data(&d3, ga3.data(), w3.data(), gr2.data());
  flref_relu_bwd((int64_t)nm, gr2.data(), n2.data(), gn2.data());
  flref_bn_bwd(N, Cm, HW, a2.data(), gn2.data(), g2.data(), m2.data(), v2.data(), 1e-5, ga2.data(), dg2.data(), db2.data());
  flref_conv2d_bwd_filter(&d2, r1.data(), ga2.data(), dw2.data(), nullptr);
  flref_conv2d_bwd_data(&d2, ga2.data(), w2.data(), gr1.data());
  flref_relu_bwd((int64_t)nm, gr1.data(), n1.data(), gn1.data());
  flref_bn_bwd(N, Cm, HW, a1.data(), gn1.data(), g1.data(), m1.data(), v1.data(), 1e-5, ga1.data(), dg1.data(), db1.data());
  flref_conv2d_bwd_filter(&d1, x.data(), ga1.data(), dw1.data(), nullptr);
  flref_conv2d_bwd_data(&d1, ga1.data(), w1.data(), gx.data());
  for (size_t i = 0; i < ni; ++i) gx[i] += gs[i];        // the residual branch
  CHECK(relL2(hostOf(in.grad()), gx) <= 2e-4);
  CHECK(relL2(hostOf(c1.param(0).grad()), dw1) <= 2e-4 && relL2(hostOf(c2.param(0).grad()), dw2) <= 2e-4 &&
        relL2(hostOf(c3.param(0).grad()), dw3) <= 2e-4);
  CHECK(relL2(hostOf(b1.param(0).grad()), dg1) <= 2e-4 && relL2(hostOf(b1.param(1).grad()), db1) <= 2e-4);
  CHECK(relL2(hostOf(b2.param(0).grad()), dg2) <= 2e-4 && relL2(hostOf(b2.param(1).grad()), db2) <= 2e-4);
  CHECK(relL2(hostOf(b3.param(0).grad()), dg3) <= 2e-4 && relL2(hostOf(b3.param(1).grad()), db3) <= 2e-4);
  CHECK(throws<std::invalid_argument>([&] { t3 + c1(in); }));   // shapes differ
}

// configs[3]: three (Conv 21x1 SAME -> BatchNorm over axis 2 -> ReLU) layers on [T, 1, 80, B],
// channels 80 -> 250 -> 250 -> 250, strides 1, 1, 2 along time, from modules; forward and
// backward against the CPU checker, at a shortened size and at the stated one (T = 1500, B = 16).
static void testSpeechStack(const int T, const int B) {
  std::printf("speech stack (21x1 convolutions, batch norm, ReLU), T = %d, batch %d\n", T, B);
  const int chans[4] = {80, 250, 250, 250}, strides[3] = {1, 1, 2};
  setSeed(17);
  std::vector<Conv2D> convs;
  std::vector<BatchNorm> bns;
  for (int l = 0; l < 3; ++l) {
    convs.emplace_back(chans[l], chans[l + 1], 21, 1, strides[l], 1, PaddingMode::SAME, PaddingMode::SAME);
    bns.emplace_back(2, chans[l + 1]);
  }
  auto x = randn((size_t)B * 80 * T, 71);
  Variable in(Tensor::fromVector({T, 1, 80, B}, x), true);
  Variable h = in;
  std::vector<Variable> preRelu;       // the device's batch-norm results: the ReLU's mask on the way back
  for (int l = 0; l < 3; ++l) {
    preRelu.push_back(bns[l](convs[l](h)));
    h = relu(preRelu.back());
  }
  const int Tout = T / 2;
  CHECK(h.shape() == Shape({Tout, 1, 250, B}));
  auto dy = randn((size_t)B * 250 * Tout, 72);
  h.backward(Variable(Tensor::fromVector(h.shape(), dy), false));

  // ---- CPU checker: keep every layer's tensors for the way back ----------------------
  struct Layer {
    flref_conv d;
    std::vector<float> in, a, n, r, w, b, g, z, mean, var;
    int64_t hw;
  };
  std::vector<Layer> L(3);
  std::vector<float> cur = x;
  int t = T;
  for (int l = 0; l < 3; ++l) {
    Layer& y = L[l];
    const int pad = derivePadding(t, 21, strides[l], -1, 1);
    y.d = flref_conv{B, chans[l], 1, t, chans[l + 1], 1, 21, 1, strides[l], 0, pad, 1, 1, 1};
    int32_t oh, ow;
    flref_conv_out(&y.d, &oh, &ow);
    y.hw = (int64_t)oh * ow;
    const size_t no = (size_t)B * chans[l + 1] * y.hw;
    y.in = cur;
    y.w = hostOf(convs[l].param(0)); y.b = hostOf(convs[l].param(1));
    y.g = hostOf(bns[l].param(0)); y.z = hostOf(bns[l].param(1));
    y.a.resize(no); y.n.resize(no); y.r.resize(no); y.mean.resize(chans[l + 1]); y.var.resize(chans[l + 1]);
    flref_conv2d_fwd(&y.d, y.in.data(), y.w.data(), y.b.data(), y.a.data());
    flref_bn_fwd_train(B, chans[l + 1], y.hw, y.a.data(), y.g.data(), y.z.data(), 1e-5, y.n.data(), y.mean.data(), y.var.data());
    flref_relu_fwd((int64_t)no, y.n.data(), y.r.data());
    cur = y.r;
    t = ow;
  }
  CHECK(t == Tout && relL2(hostOf(h), cur) <= 1e-4);
  std::vector<float> grad = dy;
  for (int l = 2; l >= 0; --l) {
    Layer& y = L[l];
    const size_t no = y.a.size();
    std::vector<float> gn(no), ga(no), dg(chans[l + 1]), dbn(chans[l + 1]), dw(y.w.size()), dbias(chans[l + 1]), gin(y.in.size());
    // The ReLU's mask is the one discontinuous step: a value within rounding of zero that falls on
    // the other side in the checker's forward pass moves a whole gradient element, and among millions
    // of elements a dozen of those are a relative error of 1e-3.  The checker therefore takes the mask
    // from the device's own batch-norm result, as the tape does (the results themselves agree to
    // 1e-4 above; every other step is continuous).
    const auto mask = hostOf(preRelu[l]);
    size_t flips = 0;
    for (size_t i = 0; i < no; ++i) flips += (mask[i] > 0.f) != (y.n[i] > 0.f);
    flref_relu_bwd((int64_t)no, grad.data(), mask.data(), gn.data());
    flref_bn_bwd(B, chans[l + 1], y.hw, y.a.data(), gn.data(), y.g.data(), y.mean.data(), y.var.data(), 1e-5, ga.data(),
                 dg.data(), dbn.data());
    flref_conv2d_bwd_filter(&y.d, y.in.data(), ga.data(), dw.data(), dbias.data());
    flref_conv2d_bwd_data(&y.d, ga.data(), y.w.data(), gin.data());
    const double eW = relL2(hostOf(convs[l].param(0).grad()), dw), eG = relL2(hostOf(bns[l].param(0).grad()), dg),
                 eB = relL2(hostOf(bns[l].param(1).grad()), dbn);
    std::printf("  layer %d: %zu of %zu mask elements differ from the checker's forward pass; dw %.2e dgamma %.2e dbeta %.2e\n",
                l, flips, no, eW, eG, eB);
    CHECK(flips <= no / 100000 + 2);
    CHECK(eW <= 3e-4);
    CHECK(eG <= 3e-4 && eB <= 3e-4);
    // the bias gradient of a convolution followed by batch norm is zero up to rounding:
    // compare it on the scale of the filter gradient
    double num = 0, den = 0;
    const auto gb = hostOf(convs[l].param(1).grad());
    for (size_t i = 0; i < gb.size(); ++i) num += ((double)gb[i] - dbias[i]) * ((double)gb[i] - dbias[i]);
    for (float v : dw) den += (double)v * v;
    CHECK(std::sqrt(num) <= 1e-4 * std::sqrt(den));
    grad = gin;
  }
  CHECK(relL2(hostOf(in.grad()), grad) <= 3e-4);
}

// Architecture lines (flashlight/pkg/runtime/common/SequentialBuilder.cpp:28-67, 98-640): a
// network built from text must be the network built by hand from the same modules - same
// parameters from the same seed, bit-identical outputs and gradients.
static void testArchBuilder() {
  std::printf("architecture lines\n");
  using fl::pkg::runtime::buildSequentialModule;
  const std::vector<std::string> arch = {
      "# speech-style stack, then a recurrent layer and a classifier",
      "",
      "  V -1 1 NFEAT 0  ",
      "C NFEAT 48 21 1 -1",
      "BN 48 2",
      "R",
      "C2 48 64 5 1 2 1 -1 0 1 1",
      "LN 0 1 2",
      "R",
      "M 2 1 2 1",
      "V 0 64 -1",
      "V 64 -1 1",      // [T, C, B] memory is not [C, T, B]: only the shapes matter to this test
      "GRU 64 32 1 1",
      "V 64 -1",
      "L 64 NLABEL 0",
      "LSM 0",
  };
  const int T = 40, F = 12, B = 3, NL = 7;
  setSeed(91);
  auto net = buildSequentialModule(arch, F, NL);
  CHECK(net->modules().size() == 14);
  setSeed(91);
  Sequential ref;
  ref.add(View(Shape({-1, 1, F, 0})));
  ref.add(Conv2D(F, 48, 21, 1, 1, 1, -1, 0, 1, 1));
  ref.add(BatchNorm(std::vector<int>{2}, 48));
  ref.add(ReLU());
  ref.add(Conv2D(48, 64, 5, 1, 2, 1, -1, 0, 1, 1));
  ref.add(LayerNorm(std::vector<int>{0, 1, 2}));
  ref.add(ReLU());
  ref.add(Pool2D(2, 1, 2, 1, 0, 0, PoolingMode::MAX));
  ref.add(View(Shape({0, 64, -1})));
  ref.add(View(Shape({64, -1, 1})));
  ref.add(RNN(64, 32, 1, RnnMode::GRU, true, 0.0f));
  ref.add(View(Shape({64, -1})));
  ref.add(Linear(64, NL, false));
  ref.add(LogSoftmax(0));
  CHECK(net->params().size() == ref.params().size());
  for (size_t i = 0; i < ref.params().size() && i < net->params().size(); ++i)
    CHECK(net->param((int)i).shape() == ref.param((int)i).shape() &&
          hostOf(net->param((int)i)) == hostOf(ref.param((int)i)));
  auto x = randn((size_t)T * F * B, 92);
  Variable in1(Tensor::fromVector({T, F, 1, B}, x), true), in2(Tensor::fromVector({T, F, 1, B}, x), true);
  Variable y1 = net->forward(in1), y2 = ref.forward(in2);
  CHECK(y1.shape() == y2.shape() && y1.shape().dim(0) == NL);
  CHECK(hostOf(y1) == hostOf(y2));
  auto dy = randn((size_t)y1.tensor().elements(), 93);
  y1.backward(Variable(Tensor::fromVector(y1.shape(), dy), false));
  y2.backward(Variable(Tensor::fromVector(y2.shape(), dy), false));
  CHECK(hostOf(in1.grad()) == hostOf(in2.grad()));
  for (size_t i = 0; i < ref.params().size() && i < net->params().size(); ++i)
    CHECK(hostOf(net->param((int)i).grad()) == hostOf(ref.param((int)i).grad()));

  // optional arguments and their defaults
  auto one = [](const std::string& l) { return buildSequentialModule(std::vector<std::string>{l}, 1, 1)->module(0); };
  CHECK(one("C 3 4 5 2")->prettyString() == Conv2D(3, 4, 5, 1, 2, 1, 0, 0, 1, 1).prettyString());
  CHECK(one("C1 3 4 5 2 1 2")->prettyString() == Conv2D(3, 4, 5, 1, 2, 1, 1, 0, 2, 1).prettyString());
  CHECK(one("C2 3 4 5 6 1 2")->prettyString() == Conv2D(3, 4, 5, 6, 1, 2, 0, 0, 1, 1).prettyString());
  CHECK(one("A 3 3 2 2 1 1")->prettyString() == Pool2D(3, 3, 2, 2, 1, 1, PoolingMode::AVG_INCLUDE_PADDING).prettyString());
  CHECK(one("L 5 6")->params().size() == 2 && one("L 5 6 0")->params().size() == 1 && one("L 5 6 1")->params().size() == 2);
  CHECK(one("LSTM 4 5 2 1")->prettyString() == RNN(4, 5, 2, RnnMode::LSTM, true, 0.0f).prettyString());
  CHECK(one("RNN 4 5")->prettyString() == RNN(4, 5, 1, RnnMode::RELU, false, 0.0f).prettyString());
  CHECK(one("BN 8 0 1")->prettyString() == BatchNorm(std::vector<int>{0, 1}, 8).prettyString());
  // malformed lines, lines for modules that do not exist here, a missing file
  for (const char* bad : {"C 3 4 5", "C2 3 4 5 6 1", "L 5", "BN 8", "LN", "LN 3", "M 2 2 2", "R 1", "LSM", "GRU 4",
                          "C 3 x 5 1", "XYZ 1 2", "RO", "DO", "DO 0.2 1", "GLU", "ELU 1", "SH 1 2", "WN 3", "WN 1 C 4 4 3 1", "WN 3 R", "PD 0 1", "PD 0 1 1 1",
                          "TDS 10 21", "AC 1 2 3", "RES 2 1", "RES 1 0 1", "SKIP 0 2", "PC", "PC f64", "PR 1 2 3", "PR x", "E 4", "E 4 5 6", "POSEMB 4 5"})
    CHECK(throws<std::invalid_argument>([&] { one(bad); }));
  CHECK(throws<std::runtime_error>([] { buildSequentialModule(std::string("/nonexistent/arch.txt"), 1, 1); }));
  // from a file
  const std::string path = "/tmp/flhip_arch_test_" + std::to_string((long)getpid()) + ".arch";
  if (FILE* f = std::fopen(path.c_str(), "w")) {
    for (const std::string& l : arch) std::fprintf(f, "%s\n", l.c_str());
    std::fclose(f);
    setSeed(91);
    auto net2 = buildSequentialModule(path, F, NL);
    CHECK(net2->modules().size() == 14 && hostOf(net2->param(0)) == hostOf(ref.param(0)));
    std::remove(path.c_str());
  } else {
    CHECK(false);
  }
}

// the element-wise modules of nn/modules/Activations.cpp, GatedLinearUnit, Dropout and Reorder, through their
// modules and architecture lines, forward and backward against the CPU checker
static void testActivationModules() {
  std::printf("activation modules, GLU, dropout, reorder\n");
  using fl::pkg::runtime::buildSequentialModule;
  auto one = [](const std::string& l) { return buildSequentialModule(std::vector<std::string>{l}, 1, 1)->module(0); };
  struct Case { const char* line; int op; double a, b; };
  const Case cases[] = {{"ELU", 0, 1.0, 0.0}, {"R6", 1, 0.0, 6.0}, {"HT", 1, -1.0, 1.0}, {"T", 2, 0.0, 0.0},
                        {"LG", 3, 0.0, 0.0}, {"SH", 4, 1.0, 0.0}, {"SH 1.5", 4, 1.5, 0.0}};
  const Shape shp({9, 5, 4, 3});
  const size_t n = 9 * 5 * 4 * 3;
  for (dtype dt : {dtype::f32, dtype::bf16, dtype::f16}) {
    const double tol = dt == dtype::f32 ? 2e-6 : 4e-3;
    for (const Case& c : cases) {
      auto x = randn(n, 700 + c.op, 3.f), dy = randn(n, 701);
      if (c.op == 3) for (auto& v : x) v = std::fabs(v) + 0.05f;
      for (auto& v : x) v = roundTo(dt, v);
      for (auto& v : dy) v = roundTo(dt, v);
      Variable in(Tensor::fromVector(shp, x).astype(dt), true);
      auto mod = one(c.line);
      Variable y = mod->forward({in})[0];
      y.backward(Variable(Tensor::fromVector(shp, dy).astype(dt), false));
      std::vector<float> yr(n), dxr(n);
      flref_act_fwd(c.op, (int64_t)n, x.data(), c.a, c.b, yr.data());
      flref_act_bwd(c.op, (int64_t)n, dy.data(), x.data(), c.a, c.b, dxr.data());
      CHECK(y.type() == dt && in.grad().type() == dt);
      CHECK(relL2(hostOf(y), yr) <= tol);
      CHECK(relL2(hostOf(in.grad()), dxr) <= tol);
    }
    // GLU along each dimension of the column-major shape: memory order [outer][2][m]
    for (int dim : {0, 1, 2}) {
      const Shape gs({8, 6, 4, 2});
      const size_t gn = 8 * 6 * 4 * 2;
      auto x = randn(gn, 710 + dim), dy = randn(gn / 2, 711);
      for (auto& v : x) v = roundTo(dt, v);
      for (auto& v : dy) v = roundTo(dt, v);
      long long m = gs.dim(dim) / 2, outer = 1;
      for (int i = 0; i < dim; ++i) m *= gs.dim(i);
      for (int i = dim + 1; i < 4; ++i) outer *= gs.dim(i);
      Variable in(Tensor::fromVector(gs, x).astype(dt), true);
      Variable y = one("GLU " + std::to_string(dim))->forward({in})[0];
      CHECK(y.shape().dim(dim) == gs.dim(dim) / 2 && (size_t)y.tensor().elements() == gn / 2);
      y.backward(Variable(Tensor::fromVector(y.shape(), dy).astype(dt), false));
      std::vector<float> yr(gn / 2), dxr(gn);
      flref_glu_fwd(outer, m, x.data(), yr.data());
      flref_glu_bwd(outer, m, dy.data(), x.data(), dxr.data());
      CHECK(relL2(hostOf(y), yr) <= tol);
      CHECK(relL2(hostOf(in.grad()), dxr) <= tol);
    }
  }
  // LeakyReLU, ThresholdReLU (no architecture line in the reference's builder), Identity
  for (dtype dt : {dtype::f32, dtype::f16}) {
    const double tol = dt == dtype::f32 ? 2e-6 : 4e-3;
    struct MCase { std::shared_ptr<Module> m; int op; double a; const char* pretty; };
    const MCase mc[] = {{std::make_shared<LeakyReLU>(0.1), 7, 0.1, "LeakyReLU (0.100000)"},
                        {std::make_shared<ThresholdReLU>(0.5), 8, 0.5, "ThresholdReLU (0.500000)"}};
    for (const MCase& c : mc) {
      auto x = randn(n, 740 + c.op, 2.f), dy = randn(n, 741);
      for (auto& v : x) v = roundTo(dt, v);
      for (auto& v : dy) v = roundTo(dt, v);
      Variable in(Tensor::fromVector(shp, x).astype(dt), true);
      Variable y = c.m->forward({in})[0];
      y.backward(Variable(Tensor::fromVector(shp, dy).astype(dt), false));
      std::vector<float> yr(n), dxr(n);
      flref_act_fwd(c.op, (int64_t)n, x.data(), c.a, 0.0, yr.data());
      flref_act_bwd(c.op, (int64_t)n, dy.data(), x.data(), c.a, 0.0, dxr.data());
      CHECK(c.m->prettyString() == c.pretty);
      CHECK(relL2(hostOf(y), yr) <= tol && relL2(hostOf(in.grad()), dxr) <= tol);
    }
    Variable idIn(Tensor::fromVector(shp, randn(n, 742)).astype(dt), false);
    auto idOut = Identity().forward({idIn, idIn});
    CHECK(idOut.size() == 2 && idOut[0].tensor().device() == idIn.tensor().device() && Identity().prettyString() == "Identity");
  }
  // PReLU (lines PR, PR n, PR n value): one parameter, or one per index of dimension 0; the parameter's gradient
  for (dtype dt : {dtype::f32, dtype::bf16}) {
    const double tol = dt == dtype::f32 ? 2e-6 : 4e-3;
    for (const char* line : {"PR", "PR 9 0.1", "PR 1 0.5"}) {
      auto x = randn(n, 730, 2.f), dy = randn(n, 731);
      for (auto& v : x) v = roundTo(dt, v);
      for (auto& v : dy) v = roundTo(dt, v);
      auto mod = one(line);
      CHECK(mod->prettyString() == "PReLU" && mod->params().size() == 1);
      const auto w = hostOf(mod->param(0));
      const size_t size = w.size();
      CHECK(size == (std::string(line) == "PR 9 0.1" ? 9u : 1u));
      CHECK(std::fabs(w[0] - (std::string(line) == "PR" ? 0.25f : std::string(line) == "PR 9 0.1" ? 0.1f : 0.5f)) < 1e-7f);
      Variable in(Tensor::fromVector(shp, x).astype(dt), true);
      mod->zeroGrad();
      Variable y = mod->forward({in})[0];
      y.backward(Variable(Tensor::fromVector(shp, dy).astype(dt), false));
      std::vector<float> wr = w;
      for (auto& v : wr) v = roundTo(dt, v);
      std::vector<float> yr(n), dxr(n), dwr(size);
      flref_prelu_fwd((int64_t)n, 9, (int64_t)size, x.data(), wr.data(), yr.data());
      flref_prelu_bwd((int64_t)n, 9, (int64_t)size, dy.data(), x.data(), wr.data(), dxr.data(), dwr.data());
      CHECK(relL2(hostOf(y), yr) <= tol);
      CHECK(relL2(hostOf(in.grad()), dxr) <= tol);
      // (bf16: the gradient passes through the parameter's cast and is rounded to bf16 there, as LayerNorm's is)
      CHECK(mod->param(0).grad().type() == dtype::f32 && relL2(hostOf(mod->param(0).grad()), dwr) <= (dt == dtype::f32 ? 1e-5 : 4e-3));
    }
  }
  CHECK(throws<std::invalid_argument>([&] { PReLU(4).forward(Variable(Tensor::fromVector({9, 2}, randn(18, 1)), false)); }));
  // Embedding (line E dim tokens): a gather of the table's columns; the gradient adds the deltas of equal indices
  {
    setSeed(33);
    auto emb = one("E 6 5");
    CHECK(emb->prettyString() == Embedding(6, 5).prettyString() && emb->params().size() == 1);
    CHECK(emb->param(0).dim(0) == 6 && emb->param(0).dim(1) == 5);
    const auto table = hostOf(emb->param(0));
    for (float v : table) CHECK(std::fabs(v) <= std::sqrt(1.0 / 6.0) + 1e-6);
    const std::vector<int32_t> ids{3, 0, 3, 4, 0, 3, 1};
    Variable in(Tensor::fromHost(Shape({7}), dtype::s32, ids.data()), false);
    emb->zeroGrad();
    auto out = std::static_pointer_cast<UnaryModule>(emb)->forward(in);
    CHECK(out.ndim() == 2 && out.dim(0) == 6 && out.dim(1) == 7);
    const auto y = hostOf(out);
    bool same = true;
    for (int i = 0; i < 7; ++i)
      for (int d = 0; d < 6; ++d) same = same && y[i * 6 + d] == table[ids[i] * 6 + d];
    CHECK(same);
    const auto g = randn(42, 17);
    out.backward(Variable(Tensor::fromVector({6, 7}, g), false));
    std::vector<float> want(30, 0.f);
    for (int i = 0; i < 7; ++i)
      for (int d = 0; d < 6; ++d) want[ids[i] * 6 + d] += g[i * 6 + d];
    CHECK(relL2(hostOf(emb->param(0).grad()), want) <= 1e-6);
    for (int d = 0; d < 6; ++d) CHECK(hostOf(emb->param(0).grad())[2 * 6 + d] == 0.f);      // token 2 never occurs
    CHECK(throws<std::invalid_argument>([&] { embedding(Variable(Tensor::fromVector({7}, randn(7, 1)), false), emb->param(0)); }));
  }
  CHECK(throws<std::invalid_argument>([&] { gatedlinearunit(Variable(Tensor::fromVector({3, 5}, randn(15, 1)), false), 0); }));
  CHECK(throws<std::invalid_argument>([&] { gatedlinearunit(Variable(Tensor::fromVector({4, 5}, randn(20, 1)), false), 2); }));

  // dropout: rate, scale, the backward pass uses the forward pass's mask, eval mode is the identity, p = 0 too
  {
    const size_t dn = 200000;
    std::vector<float> ones(dn, 1.f);
    auto dy = randn(dn, 720);
    setSeed(5);
    auto drop = one("DO 0.3");
    Variable in(Tensor::fromVector({(Dim)dn}, ones), true);
    Variable y = drop->forward({in})[0];
    y.backward(Variable(Tensor::fromVector({(Dim)dn}, dy), false));
    auto yh = hostOf(y), gh = hostOf(in.grad());
    size_t kept = 0;
    bool ok = true;
    for (size_t i = 0; i < dn; ++i) {
      if (yh[i] != 0.f) {
        ++kept;
        ok = ok && std::fabs(yh[i] - 1.f / 0.7f) < 1e-6f && std::fabs(gh[i] - dy[i] * (1.f / 0.7f)) <= 1e-6f * std::fabs(dy[i]) + 1e-12f;
      } else {
        ok = ok && gh[i] == 0.f;
      }
    }
    CHECK(ok);
    CHECK(std::fabs((double)kept / dn - 0.7) < 4 * std::sqrt(0.3 * 0.7 / dn));
    // another call draws another mask; the same seed draws the same
    Variable y2 = drop->forward({in})[0];
    CHECK(hostOf(y2) != yh);
    setSeed(5);
    CHECK(hostOf(drop->forward({in})[0]) == yh);
    drop->eval();
    CHECK(hostOf(drop->forward({in})[0]) == ones);
    CHECK(hostOf(dropout(in, 0.0)) == ones);
    CHECK(throws<std::invalid_argument>([&] { dropout(in, 1.0); }));
  }
  // RO: the Reorder module is fl::reorder
  {
    auto x = randn(2 * 3 * 4 * 5, 730);
    Variable a(Tensor::fromVector({2, 3, 4, 5}, x), true), b(Tensor::fromVector({2, 3, 4, 5}, x), true);
    Variable y1 = one("RO 2 0 3 1")->forward({a})[0], y2 = reorder(b, Shape({2, 0, 3, 1}));
    CHECK(y1.shape() == Shape({4, 2, 5, 3}) && hostOf(y1) == hostOf(y2));
    auto dy = randn(x.size(), 731);
    y1.backward(Variable(Tensor::fromVector(y1.shape(), dy), false));
    y2.backward(Variable(Tensor::fromVector(y2.shape(), dy), false));
    CHECK(hostOf(a.grad()) == hostOf(b.grad()));
  }
  // WN: the wrapped module's weight is v g / ||v||; outputs and gradients against the plain module with that weight
  // and the checker's chain rule (WeightNorm.cpp:45-72)
  for (int which = 0; which < 2; ++which) {
    setSeed(23 + which);
    auto wn = std::dynamic_pointer_cast<WeightNorm>(one(which == 0 ? "WN 3 C 6 10 5 1 -1" : "WN 0 L 12 7"));
    CHECK(wn != nullptr);
    if (!wn) continue;
    CHECK(wn->params().size() == 3);
    const Variable v = wn->param(0), g0 = wn->param(1);
    const int dim = which == 0 ? 3 : 0;
    const long long rows = v.shape().dim(dim), cols = v.tensor().elements() / rows;
    const int fast = which == 0 ? 0 : 1;
    auto vh = hostOf(v);
    // the initial g is the norm: the initial weight is v itself
    std::vector<float> nr((size_t)rows);
    flref_rownorm(rows, cols, fast, vh.data(), nr.data());
    CHECK(g0.shape().dim(dim) == rows && (long long)g0.tensor().elements() == rows && relL2(hostOf(g0), nr) <= 1e-6);
    CHECK(relL2(hostOf(wn->module()->param(0)), vh) <= 1e-6);
    // a g of its own
    auto gh = randn((size_t)rows, 750 + which, 0.3f, 1.f);
    wn->setParams(Variable(Tensor::fromVector(g0.shape(), gh), true), 1);
    std::vector<float> wr(vh.size());
    flref_weightnorm_fwd(rows, cols, fast, vh.data(), gh.data(), wr.data());
    CHECK(relL2(hostOf(wn->module()->param(0)), wr) <= 1e-6);
    const Shape ishape = which == 0 ? Shape({20, 1, 6, 2}) : Shape({12, 5});
    auto x = randn((size_t)ishape.elements(), 752);
    Variable in1(Tensor::fromVector(ishape, x), true), in2(Tensor::fromVector(ishape, x), true);
    Variable y1 = wn->forward({in1})[0];
    // the same layer with the checker's weight
    Variable wplain(Tensor::fromVector(v.shape(), wr), true);
    Variable y2 = which == 0 ? conv2d(in2, wplain, wn->param(2), 1, 1, 2, 0, 1, 1, 1) : linear(in2, wplain, wn->param(2));
    CHECK(y1.shape() == y2.shape() && relL2(hostOf(y1), hostOf(y2)) <= 1e-6);
    auto dy = randn((size_t)y1.tensor().elements(), 753);
    for (const auto& p : wn->params()) Variable(p).zeroGrad();
    y1.backward(Variable(Tensor::fromVector(y1.shape(), dy), false));
    y2.backward(Variable(Tensor::fromVector(y2.shape(), dy), false));
    CHECK(relL2(hostOf(in1.grad()), hostOf(in2.grad())) <= 1e-6);
    auto dwh = hostOf(wplain.grad());
    std::vector<float> dvr(vh.size()), dgr((size_t)rows);
    flref_weightnorm_bwd(rows, cols, fast, dwh.data(), vh.data(), gh.data(), dvr.data(), dgr.data());
    CHECK(relL2(hostOf(wn->param(0).grad()), dvr) <= 1e-5);
    CHECK(relL2(hostOf(wn->param(1).grad()), dgr) <= 1e-5);
    CHECK(wn->prettyString().rfind("WeightNorm (", 0) == 0);
  }
  CHECK(throws<std::invalid_argument>([&] { WeightNorm(Conv2D(4, 4, 3, 1), 1).forward({Variable()}); }));
  // PD: the input inside a tensor of the value, the gradient is the inner box
  {
    auto x = randn(5 * 3 * 2 * 2, 760);
    Variable in(Tensor::fromVector({5, 3, 2, 2}, x), true);
    Variable y = one("PD -1 2 1 0 0 1 3")->forward({in})[0];
    CHECK(y.shape() == Shape({8, 3, 6, 2}));
    const int64_t dims[4] = {5, 3, 2, 2};
    const int32_t before[4] = {2, 0, 1, 0}, after[4] = {1, 0, 3, 0};
    std::vector<float> yr(8 * 3 * 6 * 2), dxr(x.size());
    flref_pad_fwd(dims, before, after, -1.0, x.data(), yr.data());
    CHECK(hostOf(y) == yr);
    auto dy = randn(yr.size(), 761);
    y.backward(Variable(Tensor::fromVector(y.shape(), dy), false));
    flref_pad_bwd(dims, before, after, dy.data(), dxr.data());
    CHECK(hostOf(in.grad()) == dxr);
    CHECK(throws<std::invalid_argument>([&] { padding(Variable(Tensor::fromVector({4, 2}, randn(8, 1)), false), {{1, 1}, {0, 0}, {1, 0}}, 0.0); }));
  }
  // AC: a window that looks only ahead (future part 1, the line's default) or only back (0): against the checker's
  // convolution with twice the SAME padding, cut at the front / the back (AsymmetricConv1D.cpp:64-104)
  for (const char* line : {"AC 4 6 5 1 -1", "AC 4 6 5 1 -1 0", "AC 4 6 5 1 -1 0.5", "AC 4 6 5 1 -1 0.75"}) {
    setSeed(29);
    auto ac = one(line);
    CHECK(ac->prettyString().rfind("AsymmetricConv1D (Conv2D", 0) == 0);
    const int T = 17, Cc = 4, K = 6, k = 5, B = 3, p0 = 2;
    const double fut = std::string(line).size() > 13 ? std::stod(std::string(line).substr(14)) : 1.0;
    const int cut = (int)(std::fabs(2 * (0.5 - fut)) * p0), pad = p0 + cut;
    auto x = randn((size_t)T * Cc * B, 770), wv = hostOf(ac->param(0)), bv = hostOf(ac->param(1));
    flref_conv d{B, Cc, 1, T, K, 1, k, 1, 1, 0, pad, 1, 1, 1};
    int32_t OH, OW;
    flref_conv_out(&d, &OH, &OW);
    CHECK(OW == T + 2 * cut);
    std::vector<float> yfull((size_t)B * K * OW), yr((size_t)B * K * T);
    flref_conv2d_fwd(&d, x.data(), wv.data(), bv.data(), yfull.data());
    const int off = fut > 0.5 ? 2 * cut : 0;
    for (int r = 0; r < B * K; ++r)
      for (int t = 0; t < T; ++t) yr[(size_t)r * T + t] = yfull[(size_t)r * OW + off + t];
    Variable in(Tensor::fromVector({T, 1, Cc, B}, x), true);
    Variable y = ac->forward({in})[0];
    CHECK(y.shape() == Shape({T, 1, K, B}));
    CHECK(relL2(hostOf(y), yr) <= 1e-5);
    // the gradient of the cut: zeros where results were dropped
    auto dy = randn(yr.size(), 771);
    std::vector<float> dyfull(yfull.size(), 0.f), dxr(x.size());
    for (int r = 0; r < B * K; ++r)
      for (int t = 0; t < T; ++t) dyfull[(size_t)r * OW + off + t] = dy[(size_t)r * T + t];
    flref_conv2d_bwd_data(&d, dyfull.data(), wv.data(), dxr.data());
    y.backward(Variable(Tensor::fromVector(y.shape(), dy), false));
    CHECK(relL2(hostOf(in.grad()), dxr) <= 1e-5);
  }
  CHECK(throws<std::invalid_argument>([&] { one("AC 4 6 5 1 2"); }));
  CHECK(throws<std::invalid_argument>([&] { one("AC 4 6 5 1 -1 1.5"); }));
  // TDS: the block from its line equals the chain of its parts (TDSBlock.cpp:13-75), with and without dropout-free
  // right padding and time in the layer norm
  for (const char* line : {"TDS 3 5 4", "TDS 3 5 4 0 10 1 0"}) {
    const bool second = std::string(line).size() > 9;
    setSeed(31);
    auto tds = std::dynamic_pointer_cast<TDSBlock>(one(line));
    CHECK(tds != nullptr);
    if (!tds) continue;
    setSeed(31);
    const int C3 = 3, KS = 5, Wd = 4, LD = C3 * Wd, inner = second ? 10 : LD;
    Sequential conv, fc;
    if (second) conv.add(Padding({std::pair<int, int>{KS - 1 - 1, 1}}, 0.0));
    conv.add(Conv2D(C3, C3, KS, 1, 1, 1, second ? IntOrPadMode(0) : IntOrPadMode(PaddingMode::SAME), 0));
    conv.add(ReLU());
    fc.add(Reorder(Shape({2, 1, 0, 3})));
    fc.add(View(Shape({LD, -1, 1, 0})));
    fc.add(Linear(LD, inner));
    fc.add(ReLU());
    fc.add(Linear(inner, LD));
    fc.add(View(Shape({C3, Wd, -1, 0})));
    fc.add(Reorder(Shape({2, 1, 0, 3})));
    const std::vector<int> axes = second ? std::vector<int>{1, 2} : std::vector<int>{0, 1, 2};
    LayerNorm ln1(axes), ln2(axes);
    CHECK(tds->params().size() == conv.params().size() + fc.params().size() + ln1.params().size() + ln2.params().size());
    const int T = 11, B = 2;
    auto x = randn((size_t)T * Wd * C3 * B, 780);
    Variable in1(Tensor::fromVector({T, Wd, C3, B}, x), true), in2(Tensor::fromVector({T, Wd, C3, B}, x), true);
    Variable y1 = tds->forward({in1})[0];
    Variable h = conv.forward(in2) + in2;
    h = ln1.forward(h);
    h = fc.forward(h) + h;
    Variable y2 = ln2.forward(h);
    CHECK(y1.shape() == in1.shape() && hostOf(y1) == hostOf(y2));
    auto dy = randn(x.size(), 781);
    y1.backward(Variable(Tensor::fromVector(y1.shape(), dy), false));
    y2.backward(Variable(Tensor::fromVector(y2.shape(), dy), false));
    CHECK(hostOf(in1.grad()) == hostOf(in2.grad()));
    CHECK(tds->prettyString() == std::string("Time-Depth Separable Block (5, ") + std::to_string(inner / 3) + ", 3) [12 -> " +
                                     std::to_string(inner) + " -> 12]");
  }
  CHECK(throws<std::invalid_argument>([&] { one("TDS 3 5 4 0 0 9"); }));
  // RES: residual blocks from text against the same network written out (Residual.cpp:82-124; SequentialBuilder.cpp:498-566)
  {
    const std::vector<std::string> arch = {
        "RES 3 2 1",
        "C 4 4 3 1 -1",
        "R",
        "C 4 6 3 1 -1",
        "SKIP 0 2 0.5",              // the input joins the output of layer 1 in front of layer 2, scaled by 0.5 there
        "SKIPL 0 4 1 0.25",          // and, through a projection, the block's output
        "C 4 6 1 1",
        "T",
        "RES 1 1 2",                 // two blocks of one layer with an identity shortcut around it
        "L 6 6",
        "SKIP 0 2",
    };
    setSeed(41);
    auto net = buildSequentialModule(arch, 1, 1);
    CHECK(net->modules().size() == 3);
    auto res = std::dynamic_pointer_cast<Residual>(net->module(0));
    CHECK(res != nullptr && res->modules().size() == 4 && res->getProjectionsIndices().size() == 1);
    setSeed(41);
    Conv2D c1(4, 4, 3, 1, 1, 1, PaddingMode::SAME, 0), c2(4, 6, 3, 1, 1, 1, PaddingMode::SAME, 0), proj(4, 6, 1, 1, 1, 1, 0, 0);
    ReLU relu1;
    Tanh tanh1;
    Linear l1(6, 6), l2(6, 6);
    const int T = 9, B = 2;
    auto x = randn((size_t)T * 4 * B, 790);
    Variable in1(Tensor::fromVector({T, 1, 4, B}, x), true), in2(Tensor::fromVector({T, 1, 4, B}, x), true);
    Variable y1 = net->module(0)->forward({in1})[0];
    Variable h = c1.forward(in2);                          // layer 1
    h = relu1.forward((h + in2) * 0.5);                    // shortcut 0 -> 2, scale before layer 2
    h = c2.forward(h);                                     // layer 3
    Variable y2 = (h + proj.forward(in2)) * 0.25;          // shortcut 0 -> 4 through the projection, scale at the output
    CHECK(y1.shape() == Shape({T, 1, 6, B}) && hostOf(y1) == hostOf(y2));
    auto dy = randn((size_t)y1.tensor().elements(), 791);
    y1.backward(Variable(Tensor::fromVector(y1.shape(), dy), false));
    y2.backward(Variable(Tensor::fromVector(y2.shape(), dy), false));
    CHECK(hostOf(in1.grad()) == hostOf(in2.grad()));
    // the rest of the network: tanh, then two residual linear blocks
    auto z = randn((size_t)6 * 5, 792);
    Variable zin1(Tensor::fromVector({6, 5}, z), true), zin2(Tensor::fromVector({6, 5}, z), true);
    Variable z1 = net->module(2)->forward({net->module(1)->forward({zin1})[0]})[0];
    Variable t = tanh1.forward(zin2);
    t = l1.forward(t) + t;
    Variable z2 = l2.forward(t) + t;
    CHECK(hostOf(z1) == hostOf(z2));
    // checks of the reference's bookkeeping
    Residual r;
    r.add(ReLU());
    r.add(ReLU());
    CHECK(throws<std::invalid_argument>([&] { r.addShortcut(0, 1); }));        // to the next layer: no shortcut
    CHECK(throws<std::invalid_argument>([&] { r.addShortcut(2, 4); }));
    r.addShortcut(0, 3);
    CHECK(throws<std::invalid_argument>([&] { r.addShortcut(0, 3); }));
    r.addScale(3, 0.5f);
    CHECK(throws<std::invalid_argument>([&] { r.addScale(3, 0.5f); }));
    CHECK(throws<std::invalid_argument>([&] { r.addScale(4, 0.5f); }));
    CHECK(throws<std::invalid_argument>([&] { buildSequentialModule(std::vector<std::string>{"RES 2 0 1", "R"}, 1, 1); }));
  }
  // PC: the cast and the gradient's cast back
  {
    auto x = randn(40, 795);
    Variable in(Tensor::fromVector({8, 5}, x), true);
    Variable y = one("PC bf16")->forward({in})[0];
    CHECK(y.type() == dtype::bf16);
    std::vector<float> xr(x);
    for (auto& v : xr) v = bf16round(v);
    CHECK(hostOf(y) == xr);
    Variable z = one("PC f32")->forward({y})[0];
    CHECK(z.type() == dtype::f32 && hostOf(z) == xr);
    auto dy = randn(40, 796);
    z.backward(Variable(Tensor::fromVector({8, 5}, dy), false));
    std::vector<float> dr(dy);
    for (auto& v : dr) v = bf16round(v);
    CHECK(in.grad().type() == dtype::f32 && hostOf(in.grad()) == dr);
    CHECK(one("PC f16")->forward({in})[0].type() == dtype::f16);
  }
  // a GLU convolution block from text, as in wav2letter's architecture files
  {
    setSeed(17);
    auto net = buildSequentialModule(std::vector<std::string>{"V -1 1 NFEAT 0", "WN 3 C NFEAT 32 5 1 -1", "GLU 2", "DO 0.2",
                                                              "PD 0 2 0", "WN 3 C 16 24 3 1", "HT", "RO 2 0 3 1", "V 24 -1",
                                                              "WN 0 L 24 NLABEL", "LSM 0"},
                                     10, 6);
    CHECK(net->modules().size() == 11);
    Variable in(Tensor::fromVector({30, 10, 1, 2}, randn(600, 740)), true);
    Variable y = net->forward(in);
    CHECK(y.shape() == Shape({6, 60}));
    y.backward(Variable(Tensor::fromVector(y.shape(), randn(360, 741)), false));
    CHECK(in.grad().shape() == in.shape());
    for (const auto& p : net->params()) CHECK(p.isGradAvailable());
  }
}

// fl::SGDOptimizer (optim/SGDOptimizer.cpp:38-68): one step against the checker for every variant, parameters without
// a gradient left alone, and a small network trained on one batch until its loss has fallen
static void testSgd() {
  std::printf("SGD optimizer\n");
  struct Cfg { float mu, wd; bool nest; const char* name; };
  for (const Cfg& c : {Cfg{0.f, 0.f, false, "SGD"}, Cfg{0.9f, 0.f, false, "SGD (momentum=0.9)"},
                       Cfg{0.9f, 0.01f, false, "SGD (weight decay=0.01) (momentum=0.9)"},
                       Cfg{0.8f, 0.005f, true, "SGD (weight decay=0.005) (Nesterov momentum=0.8)"}}) {
    auto w0 = randn(3000, 800), w1 = randn(17, 801), w2 = randn(5, 802);
    Variable p0(Tensor::fromVector({30, 100}, w0), true), p1(Tensor::fromVector({17}, w1), true),
        p2(Tensor::fromVector({5}, w2), true);
    SGDOptimizer opt({p0, p1, p2}, 0.05f, c.mu, c.wd, c.nest);
    CHECK(opt.prettyString() == c.name);
    std::vector<float> v0(w0.size(), 0.f), v1(w1.size(), 0.f);
    for (int step = 0; step < 3; ++step) {
      auto g0 = randn(w0.size(), 810 + step), g1 = randn(w1.size(), 820 + step);
      opt.zeroGrad();
      p0.addGrad(Variable(Tensor::fromVector({30, 100}, g0), false));
      p1.addGrad(Variable(Tensor::fromVector({17}, g1), false));     // p2 gets no gradient
      opt.step();
      flref_sgd((int64_t)w0.size(), w0.data(), g0.data(), v0.data(), 0.05, c.mu, c.wd, c.nest);
      flref_sgd((int64_t)w1.size(), w1.data(), g1.data(), v1.data(), 0.05, c.mu, c.wd, c.nest);
      CHECK(relL2(hostOf(p0), w0) <= 2e-6 && relL2(hostOf(p1), w1) <= 2e-6 && hostOf(p2) == w2);
    }
  }
  // Adam (optim/AdamOptimizer.cpp:45-79): three steps against the checker, with and without decay
  for (float wd : {0.f, 0.05f}) {
    auto w0 = randn(3000, 830), w2 = randn(5, 832);
    Variable p0(Tensor::fromVector({30, 100}, w0), true), p2(Tensor::fromVector({5}, w2), true);
    AdamOptimizer opt({p0, p2}, 0.01f, 0.9f, 0.99f, 1e-6f, wd);
    CHECK(opt.prettyString() == (wd != 0.f ? "Adam (weight decay=0.05)" : "Adam"));
    std::vector<float> m0(w0.size(), 0.f), v0(w0.size(), 0.f);
    for (int step = 1; step <= 3; ++step) {
      auto g0 = randn(w0.size(), 840 + step);
      opt.zeroGrad();
      p0.addGrad(Variable(Tensor::fromVector({30, 100}, g0), false));
      opt.step();
      flref_adam((int64_t)w0.size(), w0.data(), g0.data(), m0.data(), v0.data(), 0.01f, 0.9f, 0.99f, 1e-6f, wd, step);
      CHECK(relL2(hostOf(p0), w0) <= 2e-6 && hostOf(p2) == w2);
    }
  }
  // training: a two-layer convolutional classifier on one batch of separable data
  {
    using fl::pkg::runtime::buildSequentialModule;
    setSeed(51);
    auto net = buildSequentialModule(std::vector<std::string>{"C2 1 8 3 3 1 1 -1 -1", "BN 8 2", "R", "M 2 2 2 2", "C2 8 16 3 3 1 1 -1 -1",
                                                              "R", "M 2 2 2 2", "V 64 -1", "L 64 4", "LSM 0"}, 1, 4);
    const int B = 32;
    std::vector<float> x((size_t)8 * 8 * B);
    std::vector<int32_t> labels(B);
    std::mt19937 gen(52);
    std::normal_distribution<float> nd(0.f, 0.3f);
    for (int b = 0; b < B; ++b) {
      labels[b] = b % 4;
      for (int i = 0; i < 64; ++i) {
        const int r = i / 8, cidx = i % 8;
        const bool on = labels[b] == 0 ? r < 4 : labels[b] == 1 ? r >= 4 : labels[b] == 2 ? cidx < 4 : cidx >= 4;
        x[(size_t)b * 64 + i] = (on ? 1.f : -1.f) + nd(gen);
      }
    }
    Variable in(Tensor::fromVector({8, 8, 1, B}, x), false);
    Variable target(Tensor::fromHost(Shape({B}), dtype::s32, labels.data()), false);
    SGDOptimizer opt(net->params(), 0.1f, 0.9f, 1e-4f);
    float first = 0.f, last = 0.f;
    for (int step = 0; step < 30; ++step) {
      opt.zeroGrad();
      Variable loss = categoricalCrossEntropy(net->forward(in), target);
      loss.backward(Variable(Tensor::full({1}, 1., dtype::f32), false));
      opt.step();
      const float l = hostOf(loss)[0];
      if (step == 0) first = l;
      last = l;
    }
    std::printf("  loss %.4f -> %.4f over 30 steps\n", first, last);
    CHECK(first > 1.0f && last < 0.1f * first);
    // the same network trained with Adam from the same initial weights
    setSeed(51);
    auto net2 = buildSequentialModule(std::vector<std::string>{"C2 1 8 3 3 1 1 -1 -1", "BN 8 2", "R", "M 2 2 2 2", "C2 8 16 3 3 1 1 -1 -1",
                                                               "R", "M 2 2 2 2", "V 64 -1", "L 64 4", "LSM 0"}, 1, 4);
    AdamOptimizer adam(net2->params(), 0.01f);
    float afirst = 0.f, alast = 0.f;
    for (int step = 0; step < 30; ++step) {
      adam.zeroGrad();
      Variable loss = categoricalCrossEntropy(net2->forward(in), target);
      loss.backward(Variable(Tensor::full({1}, 1., dtype::f32), false));
      adam.step();
      const float l = hostOf(loss)[0];
      if (step == 0) afirst = l;
      alast = l;
    }
    std::printf("  Adam: loss %.4f -> %.4f over 30 steps\n", afirst, alast);
    CHECK(afirst == first && alast < 0.1f * afirst);
  }
}

// rnn / rnnBackward through the closure and the RNN module (flashlight/fl/test/autograd/
// AutogradRnnTest.cpp:24-90 uses 2 layers, hidden 2, input 2, bidirectional; here against
// the CPU checker instead of finite differences)
static void testRnn() {
  std::printf("rnn\n");
  const RnnMode modes[4] = {RnnMode::RELU, RnnMode::TANH, RnnMode::LSTM, RnnMode::GRU};
  const int64_t expected[4] = {56, 56, 224, 168};   // AutogradRnnTest.cpp:37-49
  for (int mi = 0; mi < 4; ++mi) {
    const RnnMode mode = modes[mi];
    const int I = 2, H = 2, L = 2, B = 2, T = 3, D = 2;
    CHECK(detail::getNumRnnParams(I, H, L, mode, true) == expected[mi]);
    flref_rnn d{I, H, L, 1, (int32_t)mode, T, B};
    const int64_t n = flref_rnn_param_count(&d);
    CHECK(n == expected[mi]);
    auto w = randn((size_t)n, 80 + mi, 0.5f), x = randn((size_t)T * B * I, 90 + mi);
    auto hx = randn((size_t)L * D * B * H, 91 + mi), cx = randn(hx.size(), 92 + mi);
    auto dy = randn((size_t)T * B * D * H, 93 + mi), dhy = randn(hx.size(), 94 + mi);
    const bool lstm = mode == RnnMode::LSTM;
    std::vector<float> y(dy.size()), hy(hx.size()), cy(hx.size());
    flref_rnn_fwd(&d, x.data(), hx.data(), lstm ? cx.data() : nullptr, w.data(), y.data(), hy.data(), lstm ? cy.data() : nullptr);
    std::vector<float> dx(x.size()), dhx(hx.size()), dcx(hx.size()), dw(w.size());
    flref_rnn_bwd(&d, x.data(), hx.data(), lstm ? cx.data() : nullptr, w.data(), dy.data(), nullptr, nullptr, dx.data(),
                  dhx.data(), lstm ? dcx.data() : nullptr, dw.data());

    Variable in(Tensor::fromVector({I, B, T}, x), true), wt(Tensor::fromVector({(Dim)n}, w), true);
    Variable h0(Tensor::fromVector({H, B, L * D}, hx), true);
    Variable c0 = lstm ? Variable(Tensor::fromVector({H, B, L * D}, cx), true) : Variable();
    Variable yv, hyv, cyv;
    std::tie(yv, hyv, cyv) = rnn(in, h0, c0, wt, H, L, mode, true, 0.f);
    CHECK(yv.shape() == Shape({D * H, B, T}) && hyv.shape() == Shape({H, B, L * D}));
    CHECK(relL2(hostOf(yv), y) <= 1e-4 && relL2(hostOf(hyv), hy) <= 1e-4);
    if (lstm) CHECK(relL2(hostOf(cyv), cy) <= 1e-4); else CHECK(cyv.isEmpty());
    yv.backward(Variable(Tensor::fromVector(yv.shape(), dy), false));
    CHECK(relL2(hostOf(in.grad()), dx) <= 2e-4 && relL2(hostOf(wt.grad()), dw) <= 2e-4);
    CHECK(relL2(hostOf(h0.grad()), dhx) <= 2e-4);
    if (lstm) CHECK(relL2(hostOf(c0.grad()), dcx) <= 2e-4);

    // only the final hidden state differentiated, no initial states
    flref_rnn_bwd(&d, x.data(), nullptr, nullptr, w.data(), nullptr, dhy.data(), nullptr, dx.data(), dhx.data(),
                  lstm ? dcx.data() : nullptr, dw.data());
    Variable in2(Tensor::fromVector({I, B, T}, x), true), wt2(Tensor::fromVector({(Dim)n}, w), true);
    std::tie(yv, hyv, cyv) = rnn(in2, Variable(), Variable(), wt2, H, L, mode, true, 0.f);
    hyv.backward(Variable(Tensor::fromVector(hyv.shape(), dhy), false));
    CHECK(relL2(hostOf(in2.grad()), dx) <= 2e-4 && relL2(hostOf(wt2.grad()), dw) <= 2e-4);

    // errors of the reference (cudnn/RNN.cpp:97-133)
    Variable badw(Tensor::fromVector({(Dim)n - 1}, std::vector<float>((size_t)n - 1, 0.f)), false);
    CHECK(throws<std::invalid_argument>([&] { rnn(in2, Variable(), Variable(), badw, H, L, mode, true, 0.f); }));
    Variable badh(Tensor::fromVector({H + 1, B, L * D}, std::vector<float>((size_t)(H + 1) * B * L * D, 0.f)), false);
    CHECK(throws<std::invalid_argument>([&] { rnn(in2, badh, Variable(), wt2, H, L, mode, true, 0.f); }));
    if (!lstm) CHECK(throws<std::invalid_argument>([&] { rnn(in2, Variable(), h0, wt2, H, L, mode, true, 0.f); }));
  }
  // the module: parameter vector, one to three inputs -> as many outputs
  setSeed(23);
  RNN lstm(5, 4, 2, RnnMode::LSTM, true);
  CHECK(lstm.params().size() == 1 && lstm.param(0).elements() == detail::getNumRnnParams(5, 4, 2, RnnMode::LSTM, true));
  for (float f : hostOf(lstm.param(0))) CHECK(std::fabs(f) <= 0.5f);
  CHECK(lstm.prettyString() == "LSTM (5->8) (2-layer) (bidirectional)");
  Variable xin(Tensor::fromVector({5, 3, 6}, randn(90, 99)), true);
  Variable out = lstm(xin);
  CHECK(out.shape() == Shape({8, 3, 6}));
  auto r3 = lstm.forward(std::vector<Variable>{xin, Variable(), Variable()});
  CHECK(r3.size() == 3 && r3[1].shape() == Shape({4, 3, 4}) && r3[2].shape() == Shape({4, 3, 4}));
  out.backward(Variable(Tensor::full(out.shape(), 1., dtype::f32), false));
  CHECK(lstm.param(0).isGradAvailable() && xin.isGradAvailable());
  CHECK(throws<std::invalid_argument>([&] { lstm.forward(std::vector<Variable>{}); }));
  // dropout between layers (cudnn/RNN.cpp:83-90): training draws a fresh mask per call, the
  // backward pass reuses the mask of its forward pass, eval switches it off (RNN.cpp:74)
  RNN drop(5, 4, 2, RnnMode::GRU, false, 0.3f);
  setSeed(31);
  Variable xd(Tensor::fromVector({5, 3, 6}, randn(90, 98)), true);
  Variable d1 = drop(xd), d2 = drop(xd);
  CHECK(d1.shape() == Shape({4, 3, 6}));
  CHECK(maxAbsDiff(hostOf(d1), hostOf(d2)) > 1e-4);         // two masks
  setSeed(31);
  CHECK(maxAbsDiff(hostOf(drop(xd)), hostOf(d1)) == 0.0);   // the same seed, the same mask
  {
    // against the CPU checker with the mask of this call: the seed is the generator's next draw
    setSeed(77);
    const unsigned long long seed = nextSeed();
    setSeed(77);
    Variable yd = drop(xd);
    flref_rnn d{5, 4, 2, 0, (int32_t)RnnMode::GRU, 6, 3, 0.3f, (uint32_t)seed, (uint32_t)(seed >> 32)};
    const std::vector<float> wv = hostOf(drop.param(0)), xv = hostOf(xd);
    std::vector<float> y(4 * 3 * 6), hy(4 * 3 * 2), dxr(xv.size()), dhx(hy.size()), dwr(wv.size());
    flref_rnn_fwd(&d, xv.data(), nullptr, nullptr, wv.data(), y.data(), hy.data(), nullptr);
    CHECK(relL2(hostOf(yd), y) < 1e-5);
    const std::vector<float> dy = randn(y.size(), 97);
    flref_rnn_bwd(&d, xv.data(), nullptr, nullptr, wv.data(), dy.data(), nullptr, nullptr, dxr.data(), dhx.data(), nullptr,
                  dwr.data());
    xd.zeroGrad();
    drop.zeroGrad();
    yd.backward(Variable(Tensor::fromVector(yd.shape(), dy), false));
    CHECK(relL2(hostOf(xd.grad()), dxr) < 1e-4);
    CHECK(relL2(hostOf(drop.param(0).grad()), dwr) < 1e-4);
  }
  {
    // 16-bit storage: the same call on bf16 tensors equals the fp32 call on the rounded values,
    // rounded once more on the way out
    const int I = 6, H = 8, L = 2, T = 5, B = 3;
    const int64_t n = detail::getNumRnnParams(I, H, L, RnnMode::LSTM, true);
    std::vector<float> wv = randn((size_t)n, 61, 0.3f), xv = randn((size_t)I * B * T, 62);
    for (auto& f : wv) f = bf16round(f);
    for (auto& f : xv) f = bf16round(f);
    Variable x32(Tensor::fromVector({I, B, T}, xv), true), w32(Tensor::fromVector({(Dim)n}, wv), true);
    Variable x16(x32.tensor().astype(dtype::bf16), true), w16(w32.tensor().astype(dtype::bf16), true);
    Variable y32, h32, c32, y16, h16, c16;
    std::tie(y32, h32, c32) = rnn(x32, Variable(), Variable(), w32, H, L, RnnMode::LSTM, true, 0.f);
    std::tie(y16, h16, c16) = rnn(x16, Variable(), Variable(), w16, H, L, RnnMode::LSTM, true, 0.f);
    CHECK(y16.type() == dtype::bf16 && h16.type() == dtype::bf16 && c16.type() == dtype::bf16);
    CHECK(relL2(hostOf(Variable(y16.tensor().astype(dtype::f32), false)), hostOf(y32)) < 4e-3);
    const std::vector<float> gy = randn((size_t)y32.elements(), 63);
    std::vector<float> gyr = gy;
    for (auto& f : gyr) f = bf16round(f);
    y32.backward(Variable(Tensor::fromVector(y32.shape(), gyr), false));
    y16.backward(Variable(Tensor::fromVector(y16.shape(), gyr).astype(dtype::bf16), false));
    CHECK(x16.grad().type() == dtype::bf16 && w16.grad().type() == dtype::bf16);
    CHECK(relL2(hostOf(Variable(x16.grad().tensor().astype(dtype::f32), false)), hostOf(x32.grad())) < 4e-3);
    CHECK(relL2(hostOf(Variable(w16.grad().tensor().astype(dtype::f32), false)), hostOf(w32.grad())) < 4e-3);
  }
  drop.eval();
  Variable e1 = drop(xd), e2 = drop(xd);
  CHECK(e1.shape() == Shape({4, 3, 6}) && maxAbsDiff(hostOf(e1), hostOf(e2)) == 0.0);   // eval: no dropout
  CHECK(throws<std::invalid_argument>([&] { RNN bad(5, 4, 2, RnnMode::GRU, false, 1.0f); bad(xd); }));
}

// a crash of the host code should say where: unbuffered output and a backtrace
static void onCrash(int sig) {
  void* frames[64];
  const int n = backtrace(frames, 64);
  const char msg[] = "host test: fatal signal, backtrace:\n";
  (void)!write(2, msg, sizeof(msg) - 1);
  backtrace_symbols_fd(frames, n, 2);
  _exit(128 + sig);
}

// Kernel choice by measurement.  The options object and audit() with the checks of the reference's own tests
// (flashlight/fl/test/common/DynamicBenchmarkTest.cpp:30-118: options tried in order, no count without increment, the
// fastest option wins, host time between two audits of one option does not count); then a Conv2D layer in
// benchmark mode: every plan (the default rule and all kernel families, the declined ones struck out) is tried
// kPlanBenchCount times per pass, the winner runs from then on and gives the same bits on every later call, the
// gradients of every call during and after the timings match the CPU checker, another batch size starts the timings
// again, and with the mode off nothing is timed.
static void testDynamicBenchmark() {
  std::printf("kernel choice by measurement (createBenchmarkOptions)\n");
  DynamicBenchmark::setBenchmarkMode(true);
  {
    const size_t maxCount = 5;
    auto options = std::make_shared<DynamicBenchmarkOptions<int>>(std::vector<int>{1, 2, 3, 4, 5}, maxCount);
    CHECK(!options->timingsComplete() && options->currentOption() == 1);
    for (size_t i = 0; i < maxCount * 5; ++i) options->accumulateTimeToCurrentOption(1);
    CHECK(options->timingsComplete() && options->currentOption() == 1);
    CHECK(throws<std::invalid_argument>([&] { options->accumulateTimeToCurrentOption(1); }));
    options->reset();
    CHECK(!options->timingsComplete());
    const int before = options->currentOption();
    options->accumulateTimeToCurrentOption(3, false);
    options->accumulateTimeToCurrentOption(4, false);
    CHECK(before == options->currentOption());
    CHECK(throws<std::invalid_argument>([] { DynamicBenchmarkOptions<int>(std::vector<int>{}, 3); }));
  }
  {
    const size_t maxCount = 5;
    auto options = std::make_shared<DynamicBenchmarkOptions<int>>(std::unordered_set<int>{1, 2, 3, 4, 5}, maxCount);
    for (size_t i = 0; i < maxCount * 5; ++i) {
      if (options->currentOption() == 4) {
        options->accumulateTimeToCurrentOption(1);
      } else {
        options->accumulateTimeToCurrentOption(10 * (i + 1), false);
        options->accumulateTimeToCurrentOption(10 * (i + 1));
      }
    }
    CHECK(options->timingsComplete() && options->currentOption() == 4);
  }
  {
    // device work of three sizes: the smallest wins; host time between two audits of one option does not count
    const std::vector<int> sizes{1 << 22, 1 << 12, 1 << 24};
    auto options = std::make_shared<DynamicBenchmarkOptions<int>>(sizes, 4);
    auto bench = std::make_shared<DynamicBenchmark>(options);
    for (size_t i = 0; i < 4 * sizes.size(); ++i) {
      const int n = bench->getOptions<DynamicBenchmarkOptions<int>>()->currentOption();
      auto work = [&] {
        for (int r = 0; r < 4; ++r) Tensor::full({n}, 1.0, dtype::f32);
      };
      bench->audit(work, false);
      usleep(n == 1 << 12 ? 20000 : 1000);
      bench->audit(work);
    }
    CHECK(options->timingsComplete() && options->currentOption() == 1 << 12);
    // mode off: the function runs, nothing is recorded
    options->reset();
    DynamicBenchmark::setBenchmarkMode(false);
    int ran = 0;
    bench->audit([&] { ++ran; });
    CHECK(ran == 1 && options->countOf(0) == 0 && !DynamicBenchmark::getBenchmarkMode());
    DynamicBenchmark::setBenchmarkMode(true);
  }
  for (const dtype type : {dtype::f32, dtype::bf16}) {
    const bool lo = type == dtype::bf16;
    const int W = 14, H = 14, C = 64, K = 64;
    setSeed(41);
    Conv2D conv(C, K, 3, 3, 1, 1, PaddingMode::SAME, PaddingMode::SAME, 1, 1, true);
    const auto w = hostOf(conv.param(0)), b = hostOf(conv.param(1));
    std::vector<float> wr = w;
    if (lo)
      for (auto& v : wr) v = bf16round(v);
    const int nplans = 1 + flhip_conv2d_plan_count(FLHIP_CONV_BWD_DATA);
    const int timed = nplans * HipAutogradExtension::kPlanBenchCount;
    std::vector<float> keptDx, keptDw;
    for (const int N : {4, 6}) {                    // the second batch size starts the timings again
      auto x = randn((size_t)N * C * H * W, 43 + N), dy = randn((size_t)N * K * H * W, 47 + N);
      if (lo) {
        for (auto& v : x) v = bf16round(v);
        for (auto& v : dy) v = bf16round(v);
      }
      flref_conv d{N, C, H, W, K, 3, 3, 1, 1, 1, 1, 1, 1, 1};
      std::vector<float> dxRef(x.size()), dwRef(w.size()), dbRef(K);
      flref_conv2d_bwd_data(&d, dy.data(), wr.data(), dxRef.data());
      flref_conv2d_bwd_filter(&d, x.data(), dy.data(), dwRef.data(), dbRef.data());
      for (int it = 0; it < timed + 3; ++it) {
        Variable in(Tensor::fromVector({W, H, C, N}, x).astype(type), true);
        conv.zeroGrad();
        Variable out = conv.forward(in);
        out.backward(Variable(Tensor::fromVector(out.shape(), dy).astype(type), false));
        const auto dx = hostOf(in.grad()), dw = hostOf(conv.param(0).grad()), db = hostOf(conv.param(1).grad());
        CHECK(relL2(dx, dxRef) <= (lo ? 4e-3 : 1e-4));
        CHECK(relL2(dw, dwRef) <= 1e-4 && relL2(db, dbRef) <= 1e-4);
        if (it == timed) {
          keptDx = dx;
          keptDw = dw;
        } else if (it > timed) {
          CHECK(dx == keptDx && dw == keptDw);       // the cached choice: the same kernel, the same bits
        }
      }
    }
  }
  DynamicBenchmark::setBenchmarkMode(false);
}

int main() {
  std::setvbuf(stdout, nullptr, _IONBF, 0);
  std::signal(SIGSEGV, onCrash);
  std::signal(SIGBUS, onCrash);
  try {
    CHECK(derivePadding(56, 3, 1, -1, 1) == 1 && derivePadding(224, 7, 2, -1, 1) == 3 &&
          derivePadding(56, 1, 2, -1, 1) == 0 && derivePadding(1500, 21, 2, -1, 1) == 10 &&
          derivePadding(9, 3, 1, 4, 1) == 4);
    testRegistration();
    testConv(dtype::f32, 1, 1e-4);
    testConv(dtype::f32, 2, 1e-4);
    testConv(dtype::bf16, 1, 2e-2);
    testConv(dtype::f16, 1, 2e-2);
    testConv(dtype::f16, 2, 2e-2);
    testConvErrors();
    testBatchingInvariance();
    testPool();
    testBatchnorm();
    testGradAccumulation();
    testMnistStep();
    testSequentialMnist();
    testBatchNormModule();
    testLayerNormModule();
    testBottleneck();
    testSpeechStack(180, 3);
    testSpeechStack(1500, 16);
    testRnn();
    testArchBuilder();
    testActivationModules();
    testSgd();
    testModuleShapesAndBatching();
    testInit();
    testDynamicBenchmark();
    fl::sync();
  } catch (const std::exception& e) {
    std::printf("unexpected exception: %s\n", e.what());
    return 2;
  }
  std::printf(g_fail ? "%d check(s) FAILED\n" : "all host extension checks passed\n", g_fail);
  std::fflush(stdout);
  // a normal return: static destructors run, as in any program that links the host library
  return g_fail ? 1 : 0;
}
